"""The planner self-check tool: argument handling and the sweep's shapes (no GPU needed)."""
import os
import sys

sys.path.insert(0, os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))),
                                "fast-transformers_amd"))

from fast_transformers_amd import plan_check  # noqa: E402


def test_sweep_shapes_and_modes():
    a = plan_check.parse_args(["--widths", "64x64,32x128", "--chains", "4,1024", "--lengths", "256,65536"])
    got = list(plan_check.shapes(a))
    # 4 chains of 256 rows are too few to time, 1024 chains of 65536 too many to hold
    assert got == [(64, 64, 4, 65536), (64, 64, 1024, 256), (32, 128, 4, 65536), (32, 128, 1024, 256)]
    quick = plan_check.parse_args(["--quick"])
    assert quick.widths == [(64, 64)] and quick.chains == [8, 80, 512]
    # every forced mode only uses variables that the tool clears again
    assert plan_check.MODES["planner"] == {}
    for env in plan_check.MODES.values():
        assert set(env) <= set(plan_check.FORCING)
