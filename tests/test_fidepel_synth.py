"""CPU: the package's synthetic Fidepel writer (what bench.py loads) against the tests' own writer and restatement - same tensor names and shapes for a
configuration, a header that the safetensors reader of the tests parses, weights the restatement runs on, and the bytes-per-token count."""
import json
import struct

import torch

import fidepel_ref as R
import fidepel_synth as S


def _header(path):
    with open(path, "rb") as f:
        n = struct.unpack("<Q", f.read(8))[0]
        return json.loads(f.read(n)), 8 + n


def test_package_writer_agrees_with_the_tests_writer(pkg, tmp_path):
    fs = pkg.fidepel_synth
    size = fs.FidepelSize("tiny", 40, 61, 4, 2, 12, 8, 8, 9, 6, 2, 24, (3, 2), 16, n_layer=3, loop=(1, 2, 2))
    cfg = fs.write_synthetic_fidepel(str(tmp_path / "m"), size, seed=5)
    assert json.load(open(tmp_path / "m" / "config.json")) == cfg
    head, base = _header(tmp_path / "m" / "model.safetensors")
    mine = S.weights(cfg, seed=1)
    assert set(head) == set(mine)
    for name, t in mine.items():
        assert head[name]["shape"] == list(t.shape) and head[name]["dtype"] == "BF16", name
    from safetensors.torch import load_file
    W = load_file(str(tmp_path / "m" / "model.safetensors"))
    out = R.forward(list(range(17)), W, cfg)
    assert out.shape == (17, 61) and bool(torch.isfinite(out).all())
    # bytes one token reads: every layer RUN's projections, the chosen experts only, the shared expert, router, head, one embedding row
    per_layer = 2 * ((4 * 12 + 2 * 12 + 2 * 8 + 4) * 40 + 40 * 4 * 8 + 6 * 40 + 2 * 2 * 24 * 40 + 2 * 16 * 40)
    assert fs.weight_bytes_per_token(cfg) == 2 * (40 + 61 * 40) + 4 * per_layer


def test_bench_sizes_are_loadable_configurations(pkg):
    fs = pkg.fidepel_synth
    for s in fs.SIZES.values():
        cfg = fs.config_of(s)
        assert s.heads % s.kv_heads == 0 and s.n_expert % s.groups[0] == 0 and s.groups[1] * (s.n_expert // s.groups[0]) >= s.top
        assert len({n for n, _ in fs.tensor_shapes(cfg)}) == len(fs.tensor_shapes(cfg))
