"""The benchmark tables of the reference's three scripts, as bench.py emits them: table names,
x axis and the exact column names (`line_vals`) of
benchmarks/ops/benchmark_linear_attn.py:11-29, benchmark_decoupled_la.py:11-29 and
benchmark_varlen_linear_attn.py:18-44, here at tiny lengths."""
import math

import pytest
import torch

import bench

SIX = ["torch_la_fwd", "flash_bla_fwd", "torch_sdpa_fwd", "torch_la_bwd", "flash_bla_bwd", "torch_sdpa_bwd"]
EXPECTED = {
    "linear_attn": ("T", [1024, 4096, 16384, 32768], SIX, "B2-H16-D64"),
    "decoupled_la": ("T", [1024, 4096, 16384, 32768], SIX, "B2-H16-D64"),
    "varlen_linear_attn": ("max_seqlen", [256, 1024, 4096],
                           ["flash_padded_fwd", "varlen_fwd", "flash_padded_fwdbwd", "varlen_fwdbwd"],
                           "varlen-equal-B8-H16-D64"),
}


def test_table_specs_name_the_reference_axes_and_columns():
    assert set(bench.TABLE_SPECS) == set(EXPECTED)
    for name, (x_name, x_vals, line_vals, plot) in EXPECTED.items():
        spec = bench.TABLE_SPECS[name]
        assert (spec["x_name"], spec["x_vals"], spec["line_vals"], spec["plot_name"]) == (x_name, x_vals, line_vals, plot)
        assert spec["dtype"] == "bf16"


@pytest.mark.gpu
def test_reference_tables_at_tiny_lengths(tmp_path):
    dev = torch.device("cuda:0")
    flush = torch.empty(1 << 20, dtype=torch.int8, device=dev)
    md = tmp_path / "tables.md"
    tables = bench.reference_tables(dev, flush, str(md), x_vals=(128, 320))
    assert list(tables) == ["linear_attn", "decoupled_la", "varlen_linear_attn"]
    for name, (x_name, _, line_vals, plot) in EXPECTED.items():
        t = tables[name]
        assert t["x_name"] == x_name and t["line_vals"] == line_vals and t["plot_name"] == plot
        assert t["x_vals"] == [128, 320] and len(t["rows"]) == 2
        for row in t["rows"]:
            assert len(row) == len(line_vals)
            assert all(isinstance(x, float) and math.isfinite(x) and x > 0 for x in row)
    text = md.read_text()
    for name, (_, _, line_vals, _) in EXPECTED.items():
        assert f"**{name}**" in text
        assert " | ".join(line_vals) in text
