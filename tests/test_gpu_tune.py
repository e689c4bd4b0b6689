"""The variant tuner (the counterpart of the reference's tuning loop, apps/cpu/kernel/conv2d.py:37-83): it checks every
candidate bit for bit against the default choice, so a run is also a parity sweep over the variants of a shape."""
import os

import pytest

from unit_amd import tune

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("kwargs", [dict(), dict(prepared=True), dict(prepared=True, instances=3),
                                    dict(dtype="f16", prepared=True), dict(prepared=True, instances=-8)])
def test_tuner_runs_and_restores_the_environment(dev, tmp_path, kwargs):
    before = {k: os.environ.get(k) for k in ("UNIT_AMD_CONV_VARIANT", "UNIT_AMD_CONV_SPLITK", "UNIT_AMD_CONV_PANEL",
                                              "UNIT_AMD_CONV_NOTABLE")}
    results = tune.tune("single:1", iters=2, verbose=False, **kwargs)
    assert len(results) == 1
    r = results[0]
    assert r["layer"] == "3x3_64_64@56" and r["us"] > 0 and r["us"] <= r["default_us"]
    assert len(r["timings"]) >= 8  # candidates that ran and matched the default bit for bit
    assert before == {k: os.environ.get(k) for k in before}
    path = tmp_path / "table.inc"
    n = tune.write_table(results, str(path))
    assert n == (1 if r["variant"] >= 0 else 0)
    if n:
        fields = path.read_text().split("{")[1].split("}")[0].split(",")
        assert len(fields) == 9 and int(fields[6]) == r["variant"]
