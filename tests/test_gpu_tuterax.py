"""Tuterax on the GPU against the float64 restatement in tests/tuterax_ref.py (which processes whole sequences, with no cache, no state and no
batching): every mechanism alone, prompts against token-by-token decoding, portions down to two tokens, mixed batches, cells and state slots that are
used again, keys made loud on purpose (far back, at the causal edge, against a strong sink), a memory that must hold for hundreds of tokens, first
tokens, long decoding, odd sizes, the serving precision, graph replays, the engine's scheduler and the trace replay tool.

The error of a logits row is the root mean square of (got - want) with the mean taken off, over the row's own root mean square.
Rows computed with exact_f32 differ from the float64 restatement by f32 rounding only: nine in ten rows stay within F32_TOL, every row within F32_WORST.
(The worst rows are ill-conditioned ones, and plain f32 arithmetic in any order shows them: a read-out of a nearly empty memory whose key and query are
nearly orthogonal is a small number that the norm behind it, with its eps, does not scale away.  A wrong mechanism - a lost state, a key one position
off - moves rows by 1e-3 and more; the tests that aim at one show that first.)  BF16_TOL bounds rows of the serving precision."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import tuterax_ref as R
import tuterax_synth as S

pytestmark = pytest.mark.gpu
F32_TOL = 2e-5
F32_WORST = 3e-4
BF16_TOL = 6e-2
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def row_errs(got, want):
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    d = got - want
    d = d - d.mean(-1, keepdims=True)
    w = want - want.mean(-1, keepdims=True)
    return np.sqrt((d ** 2).mean(-1)) / np.sqrt((w ** 2).mean(-1))


def row_err(got, want):
    return float(row_errs(got, want).max())


def close(got, want):
    e = row_errs(got, want)
    return bool(e.max() <= F32_WORST and (len(e) < 10 or np.percentile(e, 90) <= F32_TOL))


def toks(n, vocab, seed):
    return torch.randint(0, vocab, (n,), generator=torch.Generator().manual_seed(seed)).tolist()


class Rig:
    """A model folder, its weights for the oracle, and contexts of the product on it."""

    def __init__(self, pkg, folder, cfg, seed=0, tweak=None, hold=False):
        self.cfg, self.W = cfg, S.weights(cfg, seed, hold=hold)
        if tweak:
            tweak(self.W)
        self.dir = S.write(folder, cfg, self.W)
        self.pkg = pkg
        self.model = pkg.Model(self.dir)

    def ctx(self, n_ctx=256, n_seq_max=4, exact=True, n_ubatch=64, graphs=True):
        return self.pkg.Context(self.model, n_ctx=n_ctx, n_batch=max(n_ctx, n_ubatch), n_ubatch=n_ubatch, n_seq_max=n_seq_max, exact_f32=exact, use_graphs=graphs)

    def ref(self, tokens, layers=False, without=()):
        taps = [] if layers else None
        out = R.forward(self.cfg, self.W, tokens, taps, without).numpy()
        return (out, np.stack([t.numpy() for t in taps])) if layers else out


def feed(ctx, tokens, start=0, seq=0, want_all=True):
    """One decode call for tokens[start:] of a sequence; returns the logits of every fed position."""
    n = len(tokens)
    assert ctx.decode(tokens, list(range(start, start + n)), seq=[seq] * n, logits=[1] * n if want_all else None) == 0
    return np.stack([ctx.logits(i) for i in range(n)]) if want_all else ctx.logits(-1)[None]


def feed_in_portions(ctx, tokens, sizes, seq=0, start=0):
    out, at, k = [], start, 0
    while at < len(tokens):
        n = min(sizes[k % len(sizes)], len(tokens) - at)
        out.append(feed(ctx, tokens[at:at + n], at, seq))
        at += n
        k += 1
    return np.concatenate(out)


def one_by_one(ctx, tokens, start=0, seq=0):
    return np.concatenate([feed(ctx, [tokens[i]], i, seq) for i in range(start, len(tokens))])


FULL = [S.delta(mlp=S.dense()),
        S.attention(mlp=S.dense(40)),
        S.channel_delta(),
        S.attention(heads=4, kv_heads=4, dim=12, vdim=12, rot_dims=12, softcap=0, mlp=None),
        S.delta(heads=2, kv_heads=1, dim=16, vdim=8, conv=2, mlp=None),
        S.channel_delta(heads=4, kv_heads=2, dim=8, vdim=24, conv=5, ranks=(3, 1), mlp=S.dense(24))]


@pytest.fixture(scope="module")
def full(pkg, tmp_path_factory):
    """Every branch in one small model: both recurrences with one and with several value heads per key head, two to five taps, attention with part and with
    all of a head turning, with and without a soft cap, layers with and without a feed-forward."""
    return Rig(pkg, tmp_path_factory.mktemp("ttx_full"), S.config(FULL), seed=3)


# ------------------------------------------------------------------------------------------ each mechanism alone
@pytest.mark.parametrize("name,layers", [
    ("attention", [S.attention()]),
    ("attention_whole_head_turns", [S.attention(rot_dims=24)]),
    ("attention_only_the_values_turn", [S.attention(rot_dims=0)]),
    ("attention_every_head_its_own_key", [S.attention(heads=3, kv_heads=3)]),
    ("attention_no_cap", [S.attention(softcap=0, scale=1.0)]),
    ("delta", [S.delta()]),
    ("delta_one_tap", [S.delta(conv=1)]),
    ("delta_every_head_its_own_key", [S.delta(heads=3, kv_heads=3, conv=2)]),
    ("channel_delta", [S.channel_delta()]),
    ("channel_delta_shared_keys", [S.channel_delta(heads=4, kv_heads=1, ranks=(1, 2))]),
    ("feed_forward", [S.attention(heads=1, kv_heads=1, dim=8, vdim=8, rot_dims=2, mlp=S.dense(88))]),
])
def test_mechanism_alone_matches_the_restatement(pkg, tmp_path, name, layers):
    rig = Rig(pkg, tmp_path / name, S.config(layers), seed=11)
    t = toks(29, rig.cfg["vocab"], 5)
    want, taps = rig.ref(t, layers=True)
    c = rig.ctx()
    c.enable_taps(True)
    got = feed(c, t)
    for r in range(taps.shape[0]):
        assert np.abs(c.layer_out(r, len(t)) - taps[r]).max() <= 1e-4 * max(1.0, np.abs(taps[r]).max()), (name, r)
    assert close(got, want)
    assert close(one_by_one(rig.ctx(), t), want)


def test_the_restatement_tells_the_attention_parts_apart(pkg, tmp_path):
    """Sink, soft cap, turned values and the causal edge each move the logits of this model by far more than the tolerance: the product can only agree with
    the restatement if it has every one of them."""
    rig = Rig(pkg, tmp_path / "parts", S.config([S.attention(scale=1.5, softcap=4.0)]), seed=12)
    t = toks(40, rig.cfg["vocab"], 6)
    want = rig.ref(t)
    for part in ("sink", "softcap", "value_turn", "causal"):
        assert row_err(rig.ref(t, without=(part,)), want) > 1e-2, part
    assert close(feed(rig.ctx(), t), want)
    assert close(feed_in_portions(rig.ctx(), t, [7, 2, 1, 11]), want)


# ------------------------------------------------------------------------------------------ prompts, single tokens, portions
def test_prompt_equals_token_by_token(full):
    t = toks(45, full.cfg["vocab"], 1)
    want = full.ref(t)
    whole = feed(full.ctx(), t)
    single = one_by_one(full.ctx(), t)
    assert close(whole, want) and close(single, want)
    assert close(single, whole)


@pytest.mark.parametrize("sizes", [[2], [3, 2, 7], [17, 2, 2, 30], [64, 5], [1, 2, 1, 9], [12, 11, 13], [31, 1, 32, 33], [1, 1, 2, 1, 3]])
def test_portions_of_any_size(full, sizes):
    """Portions shorter than the convolutions' reach (five taps: four tokens back), portions that end on and beside the 32-token steps of the recurrence
    kernels, portions above 32 that the engine cuts again."""
    t = toks(97, full.cfg["vocab"], 2)
    got = feed_in_portions(full.ctx(n_ubatch=32), t, sizes)
    assert close(got, full.ref(t))


def test_long_decoding_after_a_prompt(full):
    t = toks(300, full.cfg["vocab"], 4)
    c = full.ctx(n_ctx=320)
    got = np.concatenate([feed(c, t[:40]), one_by_one(c, t, 40)])
    assert close(got, full.ref(t))


def test_the_first_tokens_of_a_sequence(full):
    """Position 0 sees one key and the sink, the convolutions reach back into zeros, the memory is empty."""
    t = toks(4, full.cfg["vocab"], 9)
    want = full.ref(t)
    assert close(feed(full.ctx(), t), want)
    assert close(one_by_one(full.ctx(), t), want)
    assert close(feed_in_portions(full.ctx(), t, [1, 3]), want)
    assert close(feed(full.ctx(), t[:1]), want[:1])


# ------------------------------------------------------------------------------------------ batches, cells and slots used again
def test_unequal_requests_in_one_batch_equal_each_alone(full):
    V = full.cfg["vocab"]
    reqs = [toks(n, V, 120 + i) for i, n in enumerate((37, 9, 61, 1))]
    want = [full.ref(r) for r in reqs]
    c = full.ctx(n_ctx=192, n_ubatch=48)                     # (48 cells per sequence region: the 61-token request spills into its neighbours')
    at = [0] * len(reqs)
    got = [[] for _ in reqs]
    plan = [(5, 1, 30, 1), (2, 1, 2, 0), (1, 1, 29, 0), (29, 6, 0, 0), (0, 0, 0, 0)]
    while any(at[i] < len(reqs[i]) for i in range(len(reqs))):
        for step in plan:
            tk, ps, sq, owner = [], [], [], []
            for i, n in enumerate(step):
                n = min(n if n else 1, len(reqs[i]) - at[i])
                tk += reqs[i][at[i]:at[i] + n]; ps += list(range(at[i], at[i] + n)); sq += [i] * n; owner += [i] * n
                at[i] += n
            if not tk:
                continue
            assert c.decode(tk, ps, seq=sq, logits=[1] * len(tk)) == 0
            for j, i in enumerate(owner):
                got[i].append(c.logits(j))
    for i in range(len(reqs)):
        assert close(np.stack(got[i]), want[i]), i


def test_a_sequence_that_comes_back_later_in_the_batch(full):
    """Rows of one sequence in two runs of the same batch, another sequence between them: the second run must start from the state the first one left."""
    V = full.cfg["vocab"]
    a, b = toks(20, V, 83), toks(6, V, 81)
    c = full.ctx()
    tk = a[:7] + b + a[7:20]
    ps = list(range(7)) + list(range(6)) + list(range(7, 20))
    sq = [0] * 7 + [1] * 6 + [0] * 13
    assert c.decode(tk, ps, seq=sq, logits=[1] * len(tk)) == 0
    got = np.stack([c.logits(i) for i in range(len(tk))])
    assert close(np.concatenate([got[:7], got[13:]]), full.ref(a))
    assert close(got[7:13], full.ref(b))


def test_cells_and_state_slots_are_used_again(full):
    """A context with room for one request at a time: every request takes the cells and the slot its predecessor gave back - a memory or a convolution
    that kept anything of the predecessor would show at once; then two live requests, one ends and a third takes its slot beside the survivor."""
    V = full.cfg["vocab"]
    c = full.ctx(n_ctx=64, n_seq_max=2)
    for k in range(5):
        t = toks(50 + k, V, 40 + k)
        got = feed_in_portions(c, t, [13, 2, 21], seq=k % 2)
        assert close(got, full.ref(t)), k
        assert c.kv_used() == len(t)
        assert c.kv_seq_rm(k % 2, -1, -1)
        assert c.kv_used() == 0
    a, b, d = toks(30, V, 50), toks(34, V, 51), toks(28, V, 52)
    ga = feed(c, a, 0, 0)
    gb = feed(c, b[:20], 0, 1)
    assert c.kv_seq_rm(0, -1, -1)
    gd = feed(c, d, 0, 0)
    gb = np.concatenate([gb, feed(c, b[20:], 20, 1)])
    for got, t in ((ga, a), (gb, b), (gd, d)):
        assert close(got, full.ref(t))


def test_a_recurrent_sequence_cannot_be_cut_back_but_can_be_copied(full):
    t = toks(40, full.cfg["vocab"], 7)
    c = full.ctx()
    feed(c, t[:25])
    assert not c.kv_seq_rm(0, 12, -1)                           # the state has absorbed positions 12 .. 24
    c.kv_seq_cp(0, 2, 0, -1)                                    # cells and state of the whole sequence
    tail = toks(15, full.cfg["vocab"], 8)
    got0 = feed(c, t[25:], 25, 0)
    got2 = feed(c, tail, 25, 2)
    assert close(got0, full.ref(t)[25:])
    assert close(got2, full.ref(t[:25] + tail)[25:])


# ------------------------------------------------------------------------------------------ keys and memories made loud
def _loud_rig(pkg, folder, gain=6.0, d0=12, seed=4):
    """One attention layer with a nearly one-hot softmax: one unrotated coordinate of every query and key is made loud through the norm weights, so the
    score is decided by that coordinate; the cap lies above the loud scores."""
    def tweak(W):
        W["l0.mix.q.norm"][d0] *= gain
        W["l0.mix.k.norm"][d0] *= gain
    cfg = S.config([S.attention(heads=2, kv_heads=1, dim=16, vdim=16, rot_dims=8, scale=1.0, softcap=60.0)], width=48, vocab=50)
    return Rig(pkg, folder, cfg, seed=seed, tweak=tweak)


def _loud_sequence(rig, n, p0, askers, d0=12, seed=6):
    """n tokens whose keys are quiet in the loud coordinate, except ONE token at position p0 whose key is the loudest of the vocabulary; the rows in `askers`
    hold the quiet token whose query asks for it most.  A row that sees p0 gives it nearly all its weight."""
    F64, W, eps = torch.float64, rig.W, rig.cfg["norm"]["eps"]
    x = W["embed"].to(F64) * rig.cfg["embedding"]["scale"]
    k = (R.rms_unit((x @ W["l0.mix.k"].to(F64).T).reshape(-1, 1, 16), eps) * W["l0.mix.k.norm"].to(F64))[:, 0, d0]
    q = (R.rms_unit((x @ W["l0.mix.q"].to(F64).T).reshape(-1, 2, 16), eps) * W["l0.mix.q.norm"].to(F64))[:, 0, d0]
    loud = int(torch.argmax(k))
    quiet = [int(i) for i in torch.argsort(k.abs()) if int(i) != loud][:30]
    asker = max(quiet, key=lambda i: float(q[i]))
    t = [quiet[int(i)] for i in torch.randint(0, len(quiet), (n,), generator=torch.Generator().manual_seed(seed))]
    t[p0] = loud
    for r in askers:
        t[r] = asker
    return t, quiet


@pytest.mark.parametrize("p0,far", [(0, 300), (5, 250), (63, 129), (64, 448)])
def test_a_far_key_among_hundreds(pkg, tmp_path, p0, far):
    """One loud key hundreds of positions back, at the first cell, at a cell region's last and at the next region's first cell: the asking row far behind
    gives it nearly all its weight (the restatement with another token in its place changes that row outright).  Whole prompts, portions cut by the
    micro-batch, single tokens, and a prompt that ends just before the asking row."""
    rig = _loud_rig(pkg, tmp_path / "loud")
    r = p0 + far
    n = r + 7
    t, quiet = _loud_sequence(rig, n, p0, [r, r + 3])
    want = rig.ref(t)
    other = list(t)
    other[p0] = quiet[0]
    e = row_errs(rig.ref(other), want)
    assert e[r] > 0.05 and e[r + 3] > 0.05                      # (of the logits row's own spread; the mixer's share of the stream bounds it)
    n_ctx = (n + 63) // 64 * 64
    assert close(feed(rig.ctx(n_ctx=n_ctx, n_ubatch=512), t), want)
    assert close(feed_in_portions(rig.ctx(n_ctx=n_ctx, n_ubatch=128), t, [r, 2, 100]), want)    # the asking row opens a two-token portion
    assert close(feed_in_portions(rig.ctx(n_ctx=n_ctx, n_ubatch=128), t, [r + 1, 100]), want)    # ... and closes a prompt portion
    c = rig.ctx(n_ctx=n_ctx, n_ubatch=128)
    got = np.concatenate([feed_in_portions(c, t[:r - 2], [128, 3, 100]), one_by_one(c, t, r - 2)])
    assert close(got, want)


def test_the_causal_edge(pkg, tmp_path):
    """The loud key at position p0: the asking row at p0 + 1 sees it, the one at p0 - 1 must not - also when both are rows of the same batch."""
    rig = _loud_rig(pkg, tmp_path / "edge")
    for p0 in (1, 31, 32, 40):
        t, _ = _loud_sequence(rig, p0 + 12, p0, [p0 - 1, p0 + 1])
        want = rig.ref(t)
        e = row_errs(rig.ref(t, without=("causal",)), want)
        assert e[p0 - 1] > 0.3, p0
        assert close(feed(rig.ctx(), t), want)
        assert close(feed_in_portions(rig.ctx(), t, [p0, 2, 5]), want)        # the key opens a portion
        assert close(feed_in_portions(rig.ctx(), t, [p0 + 1, 2, 5]), want)    # ... and closes one
        c = rig.ctx()
        assert close(np.concatenate([feed(c, t[:max(p0 - 1, 1)]), one_by_one(c, t, max(p0 - 1, 1))]), want)


def test_a_strong_sink_takes_its_share_once(pkg, tmp_path):
    """One head's sink as large as the sum of its rows' other terms, the other head's far below them: the first head gives about half its weight away, so
    the heads enter the output in another proportion than without sinks (a common factor would vanish in the norm behind the mixer).  Leaving the sink
    out, or counting it once per split of a scan, would change nearly every row."""
    def tweak(W):
        W["l0.mix.sink"][0] = 6.0
        W["l0.mix.sink"][1] = -6.0
    rig = Rig(pkg, tmp_path / "sink", S.config([S.attention(heads=2, kv_heads=1, dim=16, vdim=16, rot_dims=8)], width=48, vocab=50), seed=4, tweak=tweak)
    t = toks(200, 50, 16)
    want = rig.ref(t)
    assert np.median(row_errs(rig.ref(t, without=("sink",)), want)) > 0.05
    assert close(feed(rig.ctx(n_ubatch=256), t), want)
    c = rig.ctx()
    assert close(np.concatenate([feed_in_portions(c, t[:120], [50, 2]), one_by_one(c, t, 120)]), want)


@pytest.mark.parametrize("kind", ["delta", "channel_delta"])
def test_a_memory_that_holds_for_hundreds_of_tokens(pkg, tmp_path, kind):
    """Decays close to one and a state with many rows (every write wipes what lay under its key): what token 60 wrote is still read 240 and more tokens later -
    the restatement with another token 60 differs there by several times the tolerance.  A state lost or rescaled at any cut - micro-batches, portions of
    two, single tokens - would show in every later row."""
    layer = S.delta(heads=2, kv_heads=1, dim=64, vdim=24, conv=3) if kind == "delta" else S.channel_delta(heads=2, kv_heads=2, dim=48, vdim=16, conv=4, ranks=(4, 4))
    rig = Rig(pkg, tmp_path / kind, S.config([layer], width=40, vocab=60), seed=14, hold=True)
    t = toks(320, 60, 15)
    want = rig.ref(t)
    other = list(t)
    other[60] = (t[60] + 1) % 60
    assert row_errs(rig.ref(other), want)[300:].min() > 2e-3
    assert close(feed(rig.ctx(n_ctx=320, n_ubatch=512), t), want)
    assert close(feed_in_portions(rig.ctx(n_ctx=320, n_ubatch=64), t, [100, 2, 33, 1]), want)
    c = rig.ctx(n_ctx=320)
    assert close(np.concatenate([feed(c, t[:10]), one_by_one(c, t, 10)]), want)


# ------------------------------------------------------------------------------------------ other sizes
@pytest.mark.parametrize("name,cfg", [
    ("ones", S.config([S.attention(heads=1, kv_heads=1, dim=2, vdim=2, rot_dims=2, mlp=S.dense(1)), S.delta(heads=1, kv_heads=1, dim=1, vdim=1, conv=1),
                       S.channel_delta(heads=1, kv_heads=1, dim=1, vdim=1, conv=2, ranks=(1, 1))], width=8, vocab=9, embed_scale=1.0)),
    ("wide_heads", S.config([S.attention(heads=4, kv_heads=2, dim=160, vdim=72, rot_dims=64, mlp=S.dense(56)), S.delta(heads=4, kv_heads=2, dim=160, vdim=72, conv=4)], width=136, vocab=301)),
    ("wide_values", S.config([S.attention(heads=2, kv_heads=1, dim=32, vdim=256, rot_dims=32), S.channel_delta(heads=2, kv_heads=1, dim=32, vdim=200, conv=3, ranks=(9, 17))], width=64, vocab=77)),
    ("very_wide_heads", S.config([S.attention(heads=2, kv_heads=1, dim=320, vdim=272, rot_dims=320), S.delta(heads=2, kv_heads=1, dim=300, vdim=40, conv=2),
                                  S.channel_delta(heads=1, kv_heads=1, dim=130, vdim=66, conv=3, ranks=(24, 8))], width=96, vocab=55)),
    ("equal_head_sizes", S.config([S.attention(heads=8, kv_heads=4, dim=64, vdim=64, rot_dims=32, mlp=S.dense(96)), S.delta(heads=4, kv_heads=4, dim=64, vdim=64, conv=4, mlp=S.dense(96)),
                                   S.channel_delta(heads=4, kv_heads=2, dim=64, vdim=64, conv=4, ranks=(16, 16))], width=128, vocab=200)),
    # heads whose keys and values do not start on 16-byte boundaries (the attention kernel's scalar-load form), a width that is no multiple of 8
    ("unaligned", S.config([S.attention(heads=3, kv_heads=3, dim=10, vdim=14, rot_dims=6, mlp=S.dense(30)), S.delta(heads=3, kv_heads=1, dim=10, vdim=14, conv=3),
                            S.channel_delta(heads=2, kv_heads=2, dim=7, vdim=9, conv=2, ranks=(3, 5))], width=44, vocab=29)),
    ("odd_width", S.config([S.delta(mlp=S.dense(30)), S.attention(heads=2, kv_heads=2, dim=6, vdim=6, rot_dims=0), S.channel_delta(mlp=S.dense(18))], width=50, vocab=33)),
    ("eight_taps", S.config([S.delta(conv=8), S.channel_delta(conv=7)], width=40, vocab=31)),
    ("only_recurrences", S.config([S.delta(mlp=S.dense(32)), S.channel_delta(mlp=S.dense(32))], width=40, vocab=31)),
    ("only_attention", S.config([S.attention(mlp=S.dense(32)), S.attention(heads=2, kv_heads=1)], width=40, vocab=31)),
])
def test_other_sizes(pkg, tmp_path, name, cfg):
    rig = Rig(pkg, tmp_path / name, cfg, seed=21)
    t = toks(70, cfg["vocab"], 13)
    want = rig.ref(t)
    got = feed_in_portions(rig.ctx(), t, [40, 2, 1, 27])
    assert close(got, want)


@pytest.mark.parametrize("seed", [101, 102, 103, 104])
def test_configurations_drawn_at_random(pkg, tmp_path, seed):
    """Five to nine layers of any kind in any order with sizes drawn from lists (head counts 1 - 32, head sizes 16 - 128, two to four taps, ranks, with and
    without feed-forward, cap and key / query rotation): a 400-token request in portions beside a short one that comes and goes in the same batches."""
    rng = np.random.default_rng(seed)

    def pick(xs):
        return xs[int(rng.integers(0, len(xs)))]

    layers = []
    for _ in range(int(rng.integers(5, 10))):
        kind = pick(["attention", "delta", "channel_delta"])
        mlp = S.dense(pick([72, 200, 328])) if rng.random() < 0.6 else None
        if kind == "attention":
            G = pick([1, 2, 4]); H = G * pick([1, 2, 4, 8]); D = pick([16, 32, 64, 128])
            layers.append(S.attention(heads=H, kv_heads=G, dim=D, vdim=pick([16, 32, 64, 96]), rot_dims=pick([0, 8, 16, D]), base=pick([1000.0, 30000.0, 500000.0]),
                                      scale=pick([0.1, 0.2, 0.3]), softcap=pick([0, 10.0, 25.0, 50.0]), mlp=mlp))
        else:
            G = pick([1, 2, 3]); H = G * pick([1, 2, 4])
            kw = dict(heads=H, kv_heads=G, dim=pick([16, 32, 64, 128]), vdim=pick([16, 32, 64, 128]), conv=pick([2, 3, 4]), mlp=mlp)
            layers.append(S.delta(**kw) if kind == "delta" else S.channel_delta(ranks=(pick([8, 24, 32]), pick([8, 24, 40])), **kw))
    cfg = S.config(layers, width=pick([136, 200, 320]), vocab=pick([300, 1021]), eps=pick([1e-5, 1e-6]), embed_scale=pick([1.0, 4.0, 12.0]))
    rig = Rig(pkg, tmp_path / "drawn", cfg, seed=seed)
    V = cfg["vocab"]
    long, short = toks(400, V, seed), toks(23, V, seed + 1)
    c = rig.ctx(n_ctx=512, n_ubatch=128)
    got_long, got_short, at = [], [], 0
    for k, n in enumerate([150, 1, 2, 97, 1, 1, 64, 84]):
        tk, ps, sq = long[at:at + n], list(range(at, at + n)), [0] * n
        if k in (1, 5):                                          # the short request rides along, whole, and leaves again
            tk, ps, sq = tk + short, ps + list(range(len(short))), sq + [1] * len(short)
        assert c.decode(tk, ps, seq=sq, logits=[1] * len(tk)) == 0
        rows = np.stack([c.logits(i) for i in range(len(tk))])
        got_long.append(rows[:n])
        if k in (1, 5):
            got_short.append(rows[n:])
            assert c.kv_seq_rm(1, -1, -1)
        at += n
    assert close(np.concatenate(got_long), rig.ref(long))
    for g in got_short:
        assert close(g, rig.ref(short))


def test_wide_outputs_with_one_to_four_rows(pkg, tmp_path):
    """A head with thousands of output columns (the embedding table read as the output head) and one to four rows takes the four-weight-rows-per-wave form
    of the weight-stream kernel: portions of 1, 3 and 4 tokens in both precisions (up to 16 rows the activations stay f32 in either)."""
    cfg = S.config([S.delta(mlp=S.dense(4104))], width=64, vocab=4099)
    rig = Rig(pkg, tmp_path / "wide", cfg, seed=17)
    t = toks(26, cfg["vocab"], 19)
    want = rig.ref(t)
    for exact in (True, False):
        got = feed_in_portions(rig.ctx(exact=exact), t, [1, 3, 4, 2])
        assert close(got, want), exact


# ------------------------------------------------------------------------------------------ serving precision, graphs
def test_serving_precision_is_close_and_takes_the_matrix_cores(full):
    """Batches round their activations to bf16 in front of every product (2^-9 per element, through six layers of a 72-wide model); the recurrences, norms
    and softmax stay f32.  Single tokens keep f32 activations."""
    t = toks(96, full.cfg["vocab"], 30)
    want = full.ref(t)
    exact = feed(full.ctx(n_ubatch=128), t)
    bf = feed(full.ctx(exact=False, n_ubatch=128), t)
    e = row_errs(bf, want)
    assert np.median(e) <= 2e-2 and np.percentile(e, 90) <= BF16_TOL, (np.median(e), np.percentile(e, 90), e.max())
    assert row_err(bf, exact) > 1e-5                              # (activations were rounded to bf16: another kernel ran)
    single = one_by_one(full.ctx(exact=False), t)
    assert close(single, want)


def test_graph_replays_equal_eager_steps(full):
    t = toks(40, full.cfg["vocab"], 31)
    outs = []
    for graphs in (True, False):
        c = full.ctx(graphs=graphs)
        feed(c, t[:8], want_all=False)
        rows = []
        for i in range(8, len(t)):
            rows.append(feed(c, [t[i]], i, want_all=False)[0])
            if i % 7 == 0:
                c.synchronize()
        outs.append(np.stack(rows))
    assert np.array_equal(outs[0], outs[1])
    assert close(outs[0], full.ref(t)[8:])


# ------------------------------------------------------------------------------------------ the engine and the tools
def test_greedy_generation_through_the_engine(pkg, full):
    """loadmodel -> chat completion through the slot scheduler, two requests side by side; the text is decimal token ids."""
    V = full.cfg["vocab"]
    e = pkg.Engine()
    try:
        st, body = e.load_model(llama_model_path=full.dir, model="ttx", ctx_len=256, n_parallel=2, ngl=100, exact_f32=True, user_prompt="", ai_prompt="", system_prompt="")
        assert st["status_code"] == 200 and not st["has_error"], (st, body)
        prompts = [toks(11, V, 60), toks(23, V, 61)]
        n_new = 12

        def greedy(p):
            seq = list(p)
            for _ in range(n_new + 1):
                seq.append(int(np.argmax(full.ref(seq)[-1])))
            return seq[len(p):]

        import threading
        out = [None, None]

        def run(i):
            res = e.chat_completion(model="ttx", messages=[{"role": "user", "content": " ".join(map(str, prompts[i]))}], max_tokens=n_new, temperature=0.0,
                                    repeat_penalty=1.0, frequency_penalty=0.0, presence_penalty=0.0)
            out[i] = res[-1]

        th = [threading.Thread(target=run, args=(i,)) for i in range(2)]
        [x.start() for x in th]
        [x.join() for x in th]
        for i in range(2):
            st, body = out[i]
            assert st["status_code"] == 200 and not st["has_error"], (st, body)
            got = [int(x) for x in body["choices"][0]["message"]["content"].split()]
            want = greedy(prompts[i])
            assert len(got) >= n_new and got[:n_new] == want[:n_new], (got, want)
    finally:
        e.close()


def test_trace_tool_with_a_pool_that_is_always_full(pkg, tmp_path):
    """Up to four live requests of unequal lengths fed in portions of changing size beside single tokens of the others, in a pool that holds exactly what
    the live requests need (each rounded up to 64 cells): a finished request's cells and state slot go to the next one at once.  Every position of every
    request is asked for and compared with the restatement, in both precisions."""
    cfg = S.config([S.delta(heads=4, kv_heads=2, dim=16, vdim=24, conv=4, mlp=S.dense(48)),
                    S.attention(heads=6, kv_heads=3, dim=16, vdim=24, rot_dims=12, mlp=S.dense(64)),
                    S.channel_delta(heads=2, kv_heads=2, dim=24, vdim=16, conv=3, ranks=(6, 10)),
                    S.attention(heads=4, kv_heads=1, dim=32, vdim=16, rot_dims=32, softcap=0)], width=88, vocab=211)
    rig = Rig(pkg, tmp_path / "pool", cfg, seed=31)
    V = cfg["vocab"]
    rng = np.random.default_rng(5)
    lengths = [150, 64, 97, 1, 33, 128, 70, 191, 2, 65]
    reqs = {f"q{i}": toks(n, V, 300 + i) for i, n in enumerate(lengths)}
    waiting, live, at = list(reqs), [], {}
    steps, need = [], 0
    while waiting or live:
        while waiting and len(live) < 4:
            r = waiting.pop(0)
            live.append(r)
            at[r] = 0
        need = max(need, sum((len(reqs[r]) + 63) // 64 * 64 for r in live))
        entries, end = [], []
        for k, r in enumerate(live):
            if len(live) > 1 and rng.random() < 0.2:
                continue                                         # a request may sit a step out
            n = int(rng.choice([1, 1, 1, 2, 3, 5, 17, 40])) if at[r] > 0 or k != 1 else len(reqs[r])
            n = min(n, len(reqs[r]) - at[r])
            entries.append({"id": r, "tokens": reqs[r][at[r]:at[r] + n], "want": list(range(n))})
            at[r] += n
            if at[r] == len(reqs[r]):
                end.append(r)
        steps.append({"step": len(steps), "entries": entries, "end": end})
        live = [r for r in live if r not in end]
    want = {r: rig.ref(t) for r, t in reqs.items()}
    for dtype in ("float32", "bfloat16"):
        out = tmp_path / dtype
        p = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", rig.dir, "--dtype", dtype, "--out", str(out), "--max-tokens", str(need)],
                           input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True, timeout=600)
        assert p.returncode == 0, p.stderr[-2000:]
        got = {r: [] for r in reqs}
        for st in steps:
            if not any(e["want"] for e in st["entries"]):
                continue
            rows = np.fromfile(out / f"{st['step']}.f32", "<f4").reshape(-1, V)
            k = 0
            for e in st["entries"]:
                got[e["id"]].append(rows[k:k + len(e["want"])])
                k += len(e["want"])
            assert k == len(rows)
        errs = np.concatenate([row_errs(np.concatenate(got[r]), want[r]) for r in reqs])
        if dtype == "float32":
            assert errs.max() <= F32_WORST and np.percentile(errs, 90) <= F32_TOL, (errs.max(), np.percentile(errs, 90))
        else:
            assert np.median(errs) <= 2e-2 and np.percentile(errs, 90) <= BF16_TOL, (np.median(errs), np.percentile(errs, 90), errs.max())
