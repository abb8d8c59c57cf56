"""CPU: the package's synthetic Tuterax writer (what bench.py loads) against the tests' own writer and restatement - same tensor names and shapes for a
configuration, a header that the safetensors reader of the tests parses, weights the restatement runs on, and the bytes-per-token count."""
import json
import struct

import torch

import tuterax_ref as R
import tuterax_synth as S


def _header(path):
    with open(path, "rb") as f:
        n = struct.unpack("<Q", f.read(8))[0]
        return json.loads(f.read(n)), 8 + n


def test_package_writer_agrees_with_the_tests_writer(pkg, tmp_path):
    ts = pkg.tuterax_synth
    size = ts.TuteraxSize("tiny", 40, 61, 4, 2, 12, 8, 6, 4, 2, 10, 6, 3, 5, 7, 24, pattern=("Dd", "A", "Cd"))
    cfg = ts.write_synthetic_tuterax(str(tmp_path / "m"), size, seed=5)
    assert json.load(open(tmp_path / "m" / "config.json")) == cfg
    head, base = _header(tmp_path / "m" / "model.safetensors")
    mine_cfg = json.loads(json.dumps(cfg))
    for lc in mine_cfg["layers"]:
        if lc["type"] == "channel_delta":
            lc["_ranks"] = [5, 7]
    mine = S.weights(mine_cfg, seed=1)
    assert set(head) == set(mine)
    for name, t in mine.items():
        assert head[name]["shape"] == list(t.shape) and head[name]["dtype"] == "BF16", name
    from safetensors.torch import load_file
    W = load_file(str(tmp_path / "m" / "model.safetensors"))
    out = R.forward(cfg, W, list(range(17)))
    assert out.shape == (17, 61) and bool(torch.isfinite(out).all())
    # bytes one token reads: the head (the embedding table), one embedding row, every layer's projections, output projection and feed-forward
    delta = (2 * 2 * 10 + 4 * 6 + 4 + 4 + 4 * 6) * 40 + 40 * 4 * 6 + 3 * 24 * 40
    attn = (4 * 12 + 2 * 12 + 2 * 8) * 40 + 40 * 4 * 8
    chan = (2 * 2 * 10 + 4 * 6 + 4 + 5 + 7) * 40 + 4 * 10 * 5 + 4 * 6 * 7 + 40 * 4 * 6 + 3 * 24 * 40
    assert ts.weight_bytes_per_token(cfg, 5, 7) == 2 * (40 + 61 * 40) + 2 * (delta + attn + chan)


def test_bench_sizes_are_loadable_configurations(pkg):
    ts = pkg.tuterax_synth
    for s in ts.SIZES.values():
        cfg = ts.config_of(s)
        assert s.heads % s.kv_heads == 0 and s.d_heads % s.d_kv_heads == 0 and s.vdim % 2 == 0 and s.rot_dims % 2 == 0 and s.rot_dims <= s.dim
        names = [n for n, _ in ts.tensor_shapes(cfg, s.rank_a, s.rank_g)]
        assert len(set(names)) == len(names)
        assert {lc["type"] for lc in cfg["layers"]} == {"attention", "delta", "channel_delta"}
