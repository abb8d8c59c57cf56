"""CPU: the package's synthetic Dinilorn writer (what bench.py loads) against the tests' own writer and restatement - same tensor names and shapes for a
configuration, a header that the safetensors reader of the tests parses, weights the restatement runs on, and the bytes-per-token count; and the
restatement's own small parts against hand-worked values."""
import json
import math
import struct

import torch

import dinilorn_ref as R
import dinilorn_synth as S


def _header(path):
    with open(path, "rb") as f:
        n = struct.unpack("<Q", f.read(8))[0]
        return json.loads(f.read(n)), 8 + n


def test_package_writer_agrees_with_the_tests_writer(pkg, tmp_path):
    ds = pkg.dinilorn_synth
    size = ds.DinilornSize("tiny", 40, 61, 4, 2, 12, 8, 4, 9, 2, 3, 10, 6, 6, 2, 24, (3, 2), 16, rel_rows=7, bias_max=30, pattern=("Rm", "A", "Bm"), loop=(1, 3, 2))
    cfg = ds.write_synthetic_dinilorn(str(tmp_path / "m"), size, seed=5)
    assert json.load(open(tmp_path / "m" / "config.json")) == cfg
    head, base = _header(tmp_path / "m" / "model.safetensors")
    mine_cfg = json.loads(json.dumps(cfg))
    for lc in mine_cfg["layers"]:
        if lc["type"] == "attention":
            lc["_rel_rows"] = 7
    mine = S.weights(mine_cfg, seed=1)
    assert set(head) == set(mine)
    for name, t in mine.items():
        assert head[name]["shape"] == list(t.shape) and head[name]["dtype"] == "BF16", name
    from safetensors.torch import load_file
    W = load_file(str(tmp_path / "m" / "model.safetensors"))
    out = R.forward(cfg, W, list(range(17)))
    assert out.shape == (17, 61) and bool(torch.isfinite(out).all())
    # bytes one token reads: every layer RUN's projections, router and shared gate, the chosen experts only, the shared expert, head, one embedding row
    moe = 6 * 40 + 2 * 3 * 24 * 40 + 3 * 16 * 40 + 40
    ret = (2 * 3 * 10 + 2 * 3 * 6) * 40 + 40 * 3 * 6 + moe
    att = (4 * 12 + 2 * 12 + 2 * 8 + 4) * 40 + 40 * 4 * 8
    two = (2 * 4 * 6 + 2 * 2 * 6 + 2 * 8 + 4 * 8) * 40 + 40 * 4 * 8 + moe
    assert ds.weight_bytes_per_token(cfg) == 2 * (40 + 61 * 40) + 2 * (ret + 2 * (att + two))


def test_bench_sizes_are_loadable_configurations(pkg):
    ds = pkg.dinilorn_synth
    for s in ds.SIZES.values():
        cfg = ds.config_of(s)
        assert s.heads % s.kv_heads == 0 and s.n_expert % s.groups[0] == 0 and s.groups[1] * (s.n_expert // s.groups[0]) >= s.top
        assert s.rot_dims % 2 == 0 and s.rot_dims <= s.dim // 2 and s.bias_max > s.rel_rows // 2
        names = [n for n, _ in ds.tensor_shapes(cfg, s.rel_rows)]
        assert len(set(names)) == len(names)
        assert {lc["type"] for lc in cfg["layers"]} == {"retention", "attention", "attention_2"}
        assert all(0.0 < d < 1.0 for lc in cfg["layers"] if lc["type"] == "retention" for d in lc["mixer"]["decay"])


def test_distance_buckets_by_hand():
    # eight rows, reach 64: distances 0 .. 3 have rows of their own; 4 .. 63 share four rows spaced evenly in ln(d / 4) / ln(16); from 64 on the last row
    got = [R.distance_bucket(n, 8, 64) for n in (0, 3, 4, 7, 8, 15, 16, 31, 32, 63, 64, 1000)]
    assert got == [0, 3, 4, 4, 5, 5, 6, 6, 7, 7, 7, 7]
    assert [R.distance_bucket(n, 7, 11) for n in (0, 2, 3, 5, 10, 11)] == [0, 2, 3, 4, 6, 6]


def test_banded_frequencies_by_hand():
    f = R.plain_frequencies(8, 10000.0)
    assert torch.allclose(f, torch.tensor([1.0, 0.1, 0.01, 0.001], dtype=torch.float64))
    # wavelengths 6.3, 63, 628, 6283 against original 1000: below 1000 / 4 kept, above 1000 / 1 slowed eightfold, between them blended
    g = R.banded_frequencies(8, 10000.0, {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 1000})
    s = (1000 / (2 * math.pi / 0.01) - 1.0) / 3.0
    assert torch.allclose(g, torch.tensor([1.0, 0.1, (1 - s) * 0.01 / 8 + s * 0.01, 0.001 / 8], dtype=torch.float64))


def test_router_by_hand():
    # six experts in three groups of two; selection bias lifts expert 5 although its own score is the lowest
    z = torch.tensor([[2.0, -1.9, 0.0, 0.0, 1.0, -3.0]], dtype=torch.float64)
    corr = torch.tensor([0.0, 0.0, 0.0, 0.0, 0.0, 1.0])
    s = torch.sigmoid(z)
    # choice scores: .881 .130 | .5 .5 | .731 1.047 -> group sums 1.011, 1.0, 1.778: groups 2 and 0 stay open
    ids, w = R.route(z, corr, 3, 3, 2)
    assert ids.tolist() == [[5, 0, 4]]
    assert torch.allclose(w, s[:, [5, 0, 4]])
    ids, _ = R.route(z, corr * 0, 2, 3, 1)                       # without the bias group 0 wins alone
    assert ids.tolist() == [[0, 1]]


def test_query_multiplier_and_extra_term_by_hand():
    t = R.query_temperature(torch.tensor([0, 3, 4, 9, 24]), 0.5, 5.0)
    assert torch.allclose(t, 1.0 + 0.5 * torch.log(torch.tensor([1.0, 1.0, 2.0, 3.0, 6.0], dtype=torch.float64)))
    s = torch.tensor([[0.0, 0.0]], dtype=torch.float64)
    w = R.softmax_one_more(s, torch.tensor([[True, True]]))
    assert torch.allclose(w, torch.tensor([[1 / 3, 1 / 3]], dtype=torch.float64))
    w = R.softmax_one_more(torch.tensor([[50.0, -50.0]], dtype=torch.float64), torch.tensor([[True, False]]))
    assert torch.allclose(w, torch.tensor([[1.0, 0.0]], dtype=torch.float64))
