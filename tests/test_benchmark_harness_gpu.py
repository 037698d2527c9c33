"""The sequence-length sweep harness: runs end to end (tiny sweep) in its three modes, prints
positive times, and what it times computes the right values on the harness's own inputs."""
import pytest
import torch

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
    times = re.findall(r"^\s*\d+\s+((?:[0-9.]+\s*)+)$", text, flags=re.M)
    assert times and all(float(v) > 0 for row in times for v in row.split())


def test_timed_variants_compute_the_oracles_values():
    from oracle import c_oracle
    from oracle.dfw_ref import dfw_reference
    from t2fw_amd import benchmark
    from t2fw_amd.functional_dfw import DFWFunction
    from t2fw_amd.functional_lfw import LFWFunction, lfw_step
    from tests.test_lfw_gpu import TOL, TOL_CHUNK, assert_close
    value, f, q, k, f_key, s = benchmark.make_inputs(4, 128, 64, 64, torch.float16, single_query=False)
    cpu = [t.cpu() for t in (value, f, q, k, f_key, s)]
    out, nxt = LFWFunction.apply(value, f, q, k, f_key, s)
    r_out, r_nxt = c_oracle.lfw_forward(*cpu)
    assert_close(out, r_out, torch.float16, "outputs", tol=TOL_CHUNK)
    assert_close(nxt, r_nxt, torch.float16, "next_state", tol=TOL_CHUNK)
    d_out, d_fin = DFWFunction.apply(q, k, value, s)
    rd_out, rd_fin = dfw_reference(cpu[2].double(), cpu[3].double(), cpu[0].double(), cpu[5].double())
    assert_close(d_out, rd_out, torch.float16, "outputs", tol=(3e-2, 2e-2))
    assert_close(d_fin, rd_fin, torch.float16, "final_state", tol=(3e-2, 2e-2))
    # the generation step the inference mode times == the first step of the sequence
    first = [t[:, 0].contiguous() for t in (value, f, q, k, f_key)]
    o1, s1 = lfw_step(*first, s.clone(), inplace=True)
    r1, rs1 = c_oracle.lfw_forward(*[t[:, :1] for t in cpu[:5]], cpu[5])
    assert_close(o1, r1[:, 0], torch.float16, "out")
    assert_close(s1, rs1, torch.float16, "state")
    # attention as the harness computes it
    a = benchmark.softmax_attention(q, k, value)
    ra = torch.softmax(cpu[2].double() @ cpu[3].double().transpose(-1, -2), -1) @ cpu[0].double()
    assert_close(a, ra, torch.float16, "attention", tol=(1e-2, 5e-3))
