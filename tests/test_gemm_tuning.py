"""The GEMM kernel-selection table: well-formed (CPU), and harmless when in effect (GPU)."""
import csv
import os

import pytest
import torch

from recurrent_drafting_amd import gemm_tuning


def test_table_is_well_formed():
    assert os.path.exists(gemm_tuning.TABLE)
    with open(gemm_tuning.TABLE) as f:
        rows = list(csv.reader(f))
    validators = {r[1]: r[2] for r in rows if r[0] == "Validator"}
    assert {"PT_VERSION", "HIP_VERSION", "HIPBLASLT_VERSION", "ROCBLAS_VERSION", "GCN_ARCH_NAME"} <= set(validators)
    assert validators["GCN_ARCH_NAME"].startswith("gfx950")
    entries = [r for r in rows if r[0] != "Validator"]
    assert len(entries) >= 200
    for op, problem, solution, time_ms in entries:
        assert op in ("GemmTunableOp_BFloat16_TN", "GemmAndBiasTunableOp_BFloat16_TN"), op
        assert problem.startswith("tn_") and float(time_ms) > 0
        assert solution == "Default" or solution.startswith(("Gemm_Hipblaslt_", "Gemm_Rocblas_"))
    # the decode step's problems: the four layer GEMMs and the head, for row counts that are multiples of 32
    for m in (704, 768, 800, 896):
        for n, k in ((12288, 4096), (4096, 4096), (22016, 4096), (4096, 11008), (32000, 4096)):
            assert any(p == f"tn_{n}_{m}_{k}_ld_{k}_{k}_{n}" for _, p, _, _ in entries), (m, n, k)


def test_load_is_a_no_op_without_a_gpu_or_when_switched_off(monkeypatch):
    monkeypatch.setattr(gemm_tuning, "_loaded", None)
    monkeypatch.setenv("RD_GEMM_TUNING", "0")
    assert gemm_tuning.load() == 0
    monkeypatch.setattr(gemm_tuning, "_loaded", None)
    monkeypatch.delenv("RD_GEMM_TUNING")
    if not torch.cuda.is_available():
        assert gemm_tuning.load() == 0
    monkeypatch.setattr(gemm_tuning, "_loaded", None)


@pytest.mark.gpu
def test_tuned_gemm_agrees_with_the_default_choice():
    import torch.cuda.tunable as tunable

    torch.manual_seed(0)
    x = torch.randn(768, 4096, device="cuda", dtype=torch.bfloat16)
    w = torch.randn(12288, 4096, device="cuda", dtype=torch.bfloat16) * 0.02
    was = tunable.is_enabled()
    tunable.enable(False)
    want = torch.nn.functional.linear(x, w).float()
    gemm_tuning._loaded = None
    n = gemm_tuning.load()
    got = torch.nn.functional.linear(x, w).float()
    assert n == 0 or tunable.is_enabled()
    # another kernel sums in another order: bf16 rounding of the result, nothing more
    assert (got - want).abs().max() <= 2e-2 * want.abs().max()
    # leave the process as it was found: the other tests run with torch's default choice
    tunable.enable(was)
    gemm_tuning._loaded = None
