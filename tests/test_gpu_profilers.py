"""GPU test of the two measuring tools whose numbers the scheduler acts on: the load-ratio sweep
(fusion/code/profile_ratio.py --measure; the reference's fusion/expr_load_ratio/*.py and
fusion/tune/fft_sgemm_1_4.py) and the GPTB block-count / launch-size sweep
(fusion/code/profile_gptb.py; the reference's fusion/code/gptb_profile.py:1-114 with the programs of
fusion/gptb_profile/).  Short ladders: what is checked is that the measuring path runs on the device
and that what it writes has the schema and the plausibility the generator relies on."""
import json
import os
import sys

import pytest

import tacker_amd as ta
from gpu_util import setup

pytestmark = pytest.mark.gpu

CODE = os.path.join(os.path.dirname(os.path.abspath(ta.__file__)), "fusion", "code")
if CODE not in sys.path:
    sys.path.insert(0, CODE)


def test_load_ratio_sweep_measures_one_pair_on_a_four_point_ladder(tmp_path):
    setup()
    import profile_ratio
    out = tmp_path / "ratio.json"
    ks = (640, 2048)
    profile_ratio.measure(str(out), stretch=1.0, launches=20, pairs=("stencil",), k_ladder=ks, ladder_points=4)
    meas = json.loads(out.read_text())
    assert meas["tiles"] == 1024 and meas["stretch"] == 1.0 and "gfx950" in meas["device"]
    pair = meas["pairs"]["tzgemm_stencil"]
    total = pair["be_total_blocks"]
    assert total == ta.stencil_blocks(512, 512, 64)          # the Creator's instance
    assert pair["be_solo_us"] > 0
    counts = profile_ratio.ladder(total, 4)
    assert len(counts) == 4 and counts[-1] == total and counts[0] == total // 64
    assert set(pair["by_k"]) == {str(k) for k in ks}
    for k in ks:
        row = pair["by_k"][str(k)]
        assert set(row) == {"blocks", "ratio", "gemm_us", "gemm_in_fused_us", "fused_us", "earned_us"}
        assert row["blocks"] in [0] + counts                  # a rung of the ladder, or nothing earns
        assert 0.0 <= row["ratio"] <= counts[-1] / 1024
        assert row["ratio"] == round(row["blocks"] / 1024, 4)
        assert row["gemm_us"] > 0 and row["gemm_in_fused_us"] > 0 and row["fused_us"] >= row["gemm_us"] * 0.9
        assert row["fused_us"] <= 2.0 * row["gemm_us"] * 1.001 or row["blocks"] == 0   # the stretch bound
        assert row["earned_us"] >= 0.0
        if row["blocks"]:
            # what it claims to earn is what the two serial launches would cost minus the fused launch
            serial = row["gemm_us"] + pair["be_solo_us"] * row["blocks"] / total
            assert abs(serial - row["fused_us"] - row["earned_us"]) <= 0.02 + 1e-3 * serial
            assert row["earned_us"] >= meas["min_gain"] * serial - 0.02
    # a longer reduction is a longer GEMM
    assert pair["by_k"]["2048"]["gemm_us"] > pair["by_k"]["640"]["gemm_us"]
    whole = pair["whole_kernel"]
    assert whole["serial_us"] > 0 and whole["fused_us"] > 0
    assert abs(whole["gain"] - whole["serial_us"] / whole["fused_us"]) < 1e-3
    assert 0.5 < whole["gain"] < 2.0
    assert ta.spin_fail_flag() == 0


def test_gptb_sweep_measures_one_kernel(tmp_path):
    setup()
    import profile_gptb
    out = tmp_path / "gptb.json"
    profile_gptb.measure(str(out), ["stencil"], launches=20)
    meas = json.loads(out.read_text())
    k = meas["kernels"]["stencil"]
    assert set(k) >= {"blocks", "blocksize", "kinfo_workgroups_per_cu", "whole_us", "whole_us_by_workgroups_per_cu",
                      "by_block_count", "largest_deviation_from_linear_from_an_eighth_up"}
    assert k["blocks"] == ta.stencil_blocks(512, 512, 64) and k["blocksize"] == 256
    assert set(k["whole_us_by_workgroups_per_cu"]) == {str(n) for n in profile_gptb.PER_CU}
    assert all(t > 0 for t in k["whole_us_by_workgroups_per_cu"].values())
    # the launch size kinfo names is within 25 % of the best one measured here
    assert k["whole_us"] <= 1.25 * min(k["whole_us_by_workgroups_per_cu"].values())
    counts = sorted(int(n) for n in k["by_block_count"])
    assert counts[-1] == k["blocks"] and len(counts) == len(profile_gptb.LADDER)
    times = [k["by_block_count"][str(n)]["us"] for n in counts]
    assert all(t > 0 for t in times)
    # more block positions never take noticeably less time (15 % for the noise of a few launches)
    assert all(later >= 0.85 * earlier for earlier, later in zip(times, times[1:])), times
    assert times[-1] > 2.0 * times[0]
    # the predictor's linear model (src/TaskManager.cu:593-600) beside every point
    for n in counts:
        assert abs(k["by_block_count"][str(n)]["predicted_us"] - k["whole_us"] * n / k["blocks"]) <= 0.02 + 0.05 * k["whole_us"]
    assert ta.spin_fail_flag() == 0
