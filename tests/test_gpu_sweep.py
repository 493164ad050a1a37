"""The sequence-length sweep (hyperattention_amd.benchmark_single_attention) run on the GPU: the printed lines
keep the format of the reference's script (benchmark_single_attention.py:109-111) and carry sane times."""
import math
import re

import pytest

pytestmark = pytest.mark.gpu

LINE = re.compile(
    r"^\[(?P<mode>fwd|bwd|fwd\+bwd)\s*\], (?P<method>flash|hyper), seq_len: (?P<n>\d+)\s*, causal: (?P<causal>True|False), "
    r"ms: (?P<q20>[0-9.]+) \((?P<q50>[0-9.]+), (?P<q80>[0-9.]+)\) \| $")


def run_sweep(capsys, argv):
    from hyperattention_amd import benchmark_single_attention as sweep
    sweep.main(argv)
    out = capsys.readouterr().out.splitlines()
    return [m.groupdict() for m in (LINE.match(line) for line in out) if m], out


@pytest.mark.parametrize("method", ["hyper", "flash"])
@pytest.mark.parametrize("no_causal", [False, True])
def test_sweep_prints_the_reference_lines(capsys, method, no_causal):
    argv = ["--attn_method", method, "--mode", "fwd", "--min_log2_seq", "11", "--max_log2_seq", "13", "--rep", "3"]
    if no_causal:
        argv.append("--no_causal")
    rows, out = run_sweep(capsys, argv)
    # the header: one "name : value" line per option, then the shape line of the reference's script
    assert any(line.startswith("attn_method") and line.rstrip().endswith(method) for line in out)
    assert f"mode: fwd, attn_method: {method}, batch_size: 1, head_size: 24, dim: 64" in out
    assert [int(r["n"]) for r in rows] == [2048, 4096, 8192], out
    for r in rows:
        assert r["mode"] == "fwd" and r["method"] == method and r["causal"] == str(not no_causal)
        q20, q50, q80 = float(r["q20"]), float(r["q50"]), float(r["q80"])
        assert all(math.isfinite(x) and x > 0 for x in (q20, q50, q80))
        assert q20 <= q50 <= q80
    med = [float(r["q50"]) for r in rows]
    assert med[0] < med[1] < med[2], f"times must grow with the sequence length: {med}"


def test_sweep_backward_modes(capsys):
    """fwd+bwd is the forward's quantiles plus the backward's (benchmark_single_attention.py:42-52)."""
    for mode in ("bwd", "fwd+bwd"):
        rows, out = run_sweep(capsys, ["--attn_method", "hyper", "--mode", mode, "--min_log2_seq", "12",
                                       "--max_log2_seq", "13", "--rep", "3"])
        assert [int(r["n"]) for r in rows] == [4096, 8192], out
        assert all(r["mode"] == mode and float(r["q50"]) > 0 for r in rows)
        assert float(rows[0]["q50"]) < float(rows[1]["q50"])
