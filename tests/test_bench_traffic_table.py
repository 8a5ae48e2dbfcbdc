"""bench.py takes the measured HBM traffic of its roofline objects from the table of the committed
counter summary; the table has to stay readable for every kernel the bench can name as dominant."""
import bench


def test_every_gemm_kernel_of_both_workloads_has_a_measured_row():
    table = bench.measured_traffic_bytes()
    gemms = ("swiglu_gate_up", "swiglu_down", "swiglu_dgrad_dh", "swiglu_dgrad_dx", "swiglu_wgrad_w13", "swiglu_wgrad_w2")
    for workload in ("cfg3", "cfg4"):
        for k in gemms:
            assert table[workload][k] > 1e8, (workload, k)
    # the accumulating weight-gradient kernels read the old gradient as well
    for k in ("swiglu_wgrad_w13", "swiglu_wgrad_w2"):
        assert table["cfg3"][k + "_accumulate"] > table["cfg3"][k]
    assert {"pack", "adamw", "adamw_packed"} <= set(table["cfg2"])


def test_measured_traffic_is_not_below_the_algorithmic_bytes():
    from piper_amd.configs import CFG3, CFG4

    table = bench.measured_traffic_bytes()
    for name, cfg in (("cfg3", CFG3), ("cfg4", CFG4)):
        alg = bench.kernel_bytes(cfg)
        for k, measured in table[name].items():
            if k in alg:
                assert measured >= 0.95 * alg[k], (name, k, measured, alg[k])
