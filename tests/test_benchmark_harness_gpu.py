"""The sequence-length sweep harness runs end to end (tiny sweep) in its three modes."""
import pytest

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("extra", [[], ["--backward"], ["--inference", "--variants", "attention,LFWFunction,DFWFunction,lfw_step"]])
def test_sweep_runs(extra, capsys):
    from t2fw_amd import benchmark
    benchmark.main(["--max-seqlen", "384", "--reps", "3", "--bsz", "4"] + extra)
    text = capsys.readouterr().out
    assert "Run time, ms" in text and "Peak memory, MB" in text
    import re
    for n in (128, 256):                                                  # one row per sequence length in each table
        assert len(re.findall(r"^\s*%d\s" % n, text, flags=re.M)) == 2, text
