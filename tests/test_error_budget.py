"""Structure of the error budget behind the stated attention tolerance (oracle/error_budget.py), on reduced sizes.

The full-size figures quoted next to the gates in tests/test_attn_gpu.py come from the same function on the full
workloads; here the claims those gates rest on are checked on sizes the CPU finishes in seconds:
the int8 step alone already produces the worst element on the outlier workload, a finer K scale does not move it, the
fp8 steps set the typical (mean) error, and on data without outliers every stage is small in absolute terms.
"""

import torch

from ksanadit_amd.workloads import make_inputs
from oracle.error_budget import STAGES, error_budget
from oracle.sdpa_ref import sdpa_ref


def test_budget_stages_add_up_to_the_emulated_scheme():
    """Stage C of the decomposition is the scheme the kernel implements: it must agree with the emulation oracle
    (full-softmax form) on the same inputs, and with SDPA as closely as that does."""
    from oracle.sage_emul_ref import sage_emul_ref

    q, k, v = make_inputs("cpu_plumbing", heads=2, seq=700)
    res = error_budget(q, k, v)
    ref = sdpa_ref(q, k, v).float()
    emul = sage_emul_ref(q, k, v, online=False).float()
    got = (emul - ref).abs().max().item()
    # the decomposition measures against float64 attention, sdpa_ref rounds to bf16: half a bf16 ulp of slack
    assert abs(got - res["C"]["max_abs"]) <= 2.0**-9 * res["ref_max"] + 1e-4
    for s in STAGES:
        assert res[s]["mean_abs"] <= res[s]["p999_abs"] <= res[s]["max_abs"]
    assert res["A"]["mean_abs"] < res["B"]["mean_abs"] < res["C"]["mean_abs"]  # each rounding adds to the typical error


def test_worst_element_on_outlier_data_is_int8_logit_noise():
    q, k, v = make_inputs("wan14b_480p", heads=1, seq=8192)
    res = error_budget(q, k, v, rows=4096)
    finer = error_budget(q, k, v, rows=4096, k_block=32)
    # the int8 stage alone reaches (almost) the full scheme's worst element ...
    assert res["A"]["max_abs"] >= 0.8 * res["C"]["max_abs"]
    # ... a K scale per 32 keys does not repair it ...
    assert finer["A"]["max_abs"] >= 0.9 * res["A"]["max_abs"]
    # ... while the typical error is set by the two fp8 roundings
    assert res["C"]["mean_abs"] >= 1.5 * res["A"]["mean_abs"]
    # and the whole budget stays inside the gate the GPU test states for this workload (0.20 max|O|)
    assert res["C"]["max_abs"] <= 0.20 * res["ref_max"]


def test_flat_attention_meets_the_absolute_bound():
    q, k, v = make_inputs("cpu_plumbing", heads=4)
    res = error_budget(q, k, v)
    assert res["C"]["max_abs"] <= 2e-2  # the north-star example bound, where |O| << 1
    assert res["C"]["row_rel_max"] <= 0.15
