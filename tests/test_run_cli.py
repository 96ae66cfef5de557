"""The self-check driver `python -m rwkv_cuda_amd.run`: argument handling on the CPU, every op's check on the GPU."""
import pytest
import torch

from rwkv_cuda_amd import run


def test_unknown_op_is_rejected():
    with pytest.raises(SystemExit):
        run.main(["wkv9"])


@pytest.mark.skipif(torch.cuda.is_available(), reason="only meaningful without a GPU")
def test_refuses_to_run_without_a_device():
    with pytest.raises(SystemExit, match="needs a HIP device"):
        run.main(["wkv6_state", "check"])


def test_formulas_agree_with_each_other_on_cpu():
    """The driver's torch formulas are checked against one another where the ops coincide: wkv6 with a
    time-constant decay is wkv5; wkv5a with a neutral second side is wkv5."""
    torch.manual_seed(0)
    B, T, H = 2, 9, 1
    C = H * run.N
    r, k, v = (torch.rand(B, T, C) * 2 - 1 for _ in range(3))
    w, u = torch.rand(H, run.N) * 2 - 1, torch.rand(H, run.N) * 2 - 1
    dec = torch.exp(-torch.exp(w))
    y5 = run.formula_wkv(B, T, C, H, r, k, v, dec, u)
    y6 = run.formula_wkv(B, T, C, H, r, k, v, dec.reshape(1, 1, H, run.N).expand(B, T, H, run.N), u)
    y5a = run.formula_wkv(B, T, C, H, r, k, v, dec, u, None, torch.ones(H, run.N), torch.zeros(H, run.N))
    assert torch.allclose(y5, y6, atol=1e-6) and torch.allclose(y5, y5a, atol=1e-6)
    # depthwise_conv1d: out[t] = eps + sum_{u<=t} w[T-1-(t-u)] k[u]
    Tt, Cc = 8, 3
    wt, kt = torch.rand(Cc, Tt), torch.rand(1, Cc, Tt)
    out = run.formula_timex(wt, kt, 1, Cc, Tt, 0.5)
    t = 5
    want = 0.5 + sum(wt[1, Tt - 1 - (t - s)] * kt[0, 1, s] for s in range(t + 1))
    assert abs(float(out[0, 1, t]) - float(want)) < 1e-5


@pytest.mark.gpu
@pytest.mark.parametrize("op", run.OPS)
def test_check_job_passes_for_every_op(lib, op):
    print(f"\nself-check {op}", flush=True)
    lines = []
    worst, bar = run.check(op, torch.device("cuda:0"), 2, 64, 2, out=lines.append)
    print("\n".join(lines), flush=True)
    assert worst <= bar, f"{op}: worst err ratio {worst:.3e} over {bar:.0e}"


@pytest.mark.gpu
def test_benchmark_job_prints_the_profiler_tables(lib):
    lines = []
    run.benchmark("wkv6_state", torch.device("cuda:0"), 2, 256, 2, out=lines.append)
    text = "\n".join(lines)
    assert "HIP forward" in text and "HIP backward" in text


def test_head_size_option_is_validated():
    with pytest.raises(SystemExit):
        run.main(["rwkv7", "check", "--N", "4"])          # rwkv7 has head size 64 only
    with pytest.raises(SystemExit):
        run.main(["wkv6", "check", "--N", "129"])


@pytest.mark.gpu
@pytest.mark.parametrize("op,n", [("wkv6_state", 4), ("wkv6", 4), ("wkv5", 2), ("wkv5_bf16", 128), ("wkv5a", 4)])
def test_check_job_at_the_reference_drivers_head_sizes(lib, op, n):
    """The head sizes the reference's own check jobs use (wkv6_state/run.py:39, wkv6/run.py:35, wkv5/run.py:366,
    wkv5_bf16/run.py:21, wkv5a/run.py:43)."""
    old = run.N
    try:
        assert run.main([op, "check", "--N", str(n), "--T", "40"]) == 0
    finally:
        run.N = old
