"""The launch rules, grids and plans on a device of another size. Every threshold of the rules was measured on 256
compute units and is scaled by the device's own number; dlspm_tuning.compute_units makes the library size everything as
for a device of n compute units (a partition of an MI355X has 32 ... 128, other parts of the family 304), so that what
such a device would launch can be tested where there is none: results must be right for any n."""
import numpy as np
import pytest

from test_cut_plan import cut_list_offset, cut_model, dev, model, rows_with_giants, sizes  # noqa: F401 (model: a fixture)


def test_compute_units_field_scales_the_rules(dl):
    own = dl.device_info()["compute_units"]
    for bad in (1, 7, 12, 2048, -8):
        with pytest.raises(dl.DlspmError):
            dl.set_tuning(compute_units=bad)
    try:
        for cus in (32, 64, 304):
            dl.set_tuning(compute_units=cus)
            assert dl.get_tuning()["compute_units"] == cus and dl.device_info()["compute_units"] == cus
            # fewer rows than two per compute unit: eight waves per row in SDDMM from about a hundred nonzeros per row on
            assert dl.describe_launch(dl.OP_SDDMM, 2 * cus - 1, 2304, 64, (2 * cus - 1) * 200)["W"] == 8
            assert dl.describe_launch(dl.OP_SDDMM, 2 * cus, 2304, 64, 2 * cus * 200)["W"] == 4
            # rows are grouped only while the grid keeps eight workgroups per compute unit (SpMM)
            rows = lambda M: dl.describe_launch(dl.OP_SPMM, M, 1024, 64, M * 20)["R"]
            assert rows(8 * cus) == 1 and rows(16 * cus) == 2 and rows(64 * cus) == 8
            # a cut plan has room for one entry more per compute unit (bins: at most 256) and its advice follows the share
            bins = min(cus, 256)
            assert dl.row_plan_bytes_for(dl.OP_SDDMM, 1000, 0) >= 4 * 4 * (1000 + bins)
            assert dl.row_plan_advice(dl.OP_SDDMM, 1024, 2048, 128, 100000, 1 + 2 * 100000 // bins) == 2
    finally:
        dl.set_tuning()
    assert dl.device_info()["compute_units"] == own and dl.get_tuning()["compute_units"] == 0


@pytest.mark.gpu
@pytest.mark.parametrize("cus", [32, 64, 128, 304])
def test_gpu_plans_and_launches_as_on_another_device_size(model, dl, oracle, cus):
    """The device-built row and cut plans equal their sequential definitions with one bin per (pretended) compute unit, and
    all three ops -- plain, with the plan dlspm_advise asks for, and with a cut plan -- agree with the CPU oracle."""
    import torch

    rng = np.random.default_rng(cus)
    bins = min(cus, 256)
    rel = oracle.rel_frobenius
    try:
        dl.set_tuning(compute_units=cus)
        for name, M, K, mean, giants, giant_len, width in (("giants", 700, 2048, 60, 6, 1800, 128), ("lognormal", 1500, 1024, 40, 0, 0, 96),
                                                           ("few rows", 48, 1024, 300, 1, 1000, 256)):
            ro, ci = rows_with_giants(rng, M, K, mean, giants, giant_len)
            nnz = int(ci.size)
            print(f"as on {cus} compute units: {name} {M}x{K} nnz {nnz} width {width}", flush=True)
            ro_d, ci_d = dev(torch, ro), dev(torch, ci)
            # the cut plan against its definition
            E, max_cut = sizes(M, bins)
            cp = dl.cut_plan(ro_d, dl.OP_SPMM, width)
            got = cp.memory.cpu().numpy()
            want, cut, *_ = cut_model(model, ro, bins)
            assert np.array_equal(got[:4 * E], want), (name, np.flatnonzero(got[:4 * E] != want)[:10])
            assert np.array_equal(got[cut_list_offset(M, bins):][:4 + 4 * max_cut], cut), name
            # the three ops: NULL, as advised, with the cut plan
            va = rng.standard_normal(nnz).astype(np.float32)
            B = rng.standard_normal((K, width)).astype(np.float32)
            Q = rng.standard_normal((M, width)).astype(np.float32)
            V = rng.standard_normal((K, width)).astype(np.float32)
            va_d, B_d, Q_d, V_d = dev(torch, va), dev(torch, B), dev(torch, Q), dev(torch, V)
            info = dl.analyze(ro_d, ci_d, K)
            want_spmm = oracle.spmm(ro, ci, va, B, omp=True)
            want_sddmm = oracle.sddmm(ro, ci, Q, B)
            want_fused = oracle.fused(ro, ci, Q, B, V, 0.125)
            for how in ("null", "advised", "cut"):
                plans = {}
                for op in (dl.OP_SPMM, dl.OP_SDDMM, dl.OP_FUSED):
                    plans[op] = None if how == "null" else dl.prepare(ro_d, ci_d, K, op, width, info=info) if how == "advised" \
                        else dl.cut_plan(ro_d, op, width)
                assert rel(dl.spmm(ro_d, ci_d, va_d, B_d, K=K, plan=plans[dl.OP_SPMM]).cpu().numpy(), want_spmm) <= 1e-4, (name, how)
                assert rel(dl.sddmm(ro_d, ci_d, Q_d, B_d, plan=plans[dl.OP_SDDMM]).cpu().numpy(), want_sddmm) <= 1e-4, (name, how)
                assert rel(dl.fused(ro_d, ci_d, Q_d, B_d, V_d, 0.125, plan=plans[dl.OP_FUSED]).cpu().numpy(), want_fused) <= 1e-4, (name, how)
                assert np.array_equal(ro_d.cpu().numpy(), ro) and np.array_equal(ci_d.cpu().numpy(), ci)
    finally:
        dl.set_tuning()
