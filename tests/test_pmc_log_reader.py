"""The profiler-output reader (the twin of the reference's pmc_log_reader.py) on small CSV files in the
format rocprofv3 writes: kernel families by name, Gflops from the shape in a generated kernel's name,
library kernels priced with the same shape, counters averaged per dispatch."""
import csv

from codegendemo_amd.kcg import pmc_log_reader as plr

KCG = "GEMM_MNK1024x512x256_DTabcfloat32xfloat32xfloat32_AT0_TTmn4x4_BTmnk64x64x16_"
LIB = "Cijk_Ailk_Bljk_S_B_Bias_HA_S_SAV_UserArgs_MT128x128x64_MI16x16x1_"
OTHER = "void at::native::vectorized_elementwise_kernel<4, at::native::FillFunctor<float> >(int)"


def _write(path, header, rows):
    with open(path, "w", newline="") as fh:
        w = csv.writer(fh, quoting=csv.QUOTE_NONNUMERIC)
        w.writerow(header)
        w.writerows(rows)


def test_families_and_shape_from_name():
    assert plr.kernel_family(KCG) == "kcg" and plr.kernel_family(LIB) == "torch" and plr.kernel_family(OTHER) is None
    assert plr.flops_from_name(KCG) == 2 * 1024 * 512 * 256
    assert plr.flops_from_name(LIB) is None


def test_trace_and_counters(tmp_path, capsys):
    d = tmp_path / "out" / "trace"
    d.mkdir(parents=True)
    _write(d / "run_kernel_trace.csv", ["Kind", "Kernel_Name", "Start_Timestamp", "End_Timestamp"],
           [["KERNEL_DISPATCH", OTHER, 10, 20],
            ["KERNEL_DISPATCH", KCG, 1000, 3000],          # 2000 ns
            ["KERNEL_DISPATCH", LIB, 4000, 8000],          # 4000 ns
            ["KERNEL_DISPATCH", KCG, 9000, 10000]])        # 1000 ns
    p = tmp_path / "out" / "pmc"
    p.mkdir()
    _write(p / "run_counter_collection.csv", ["Dispatch_Id", "Kernel_Name", "Counter_Name", "Counter_Value"],
           [[1, KCG, "SQ_INSTS_MFMA", 100.0], [1, KCG, "SQ_LDS_BANK_CONFLICT", 0.0],
            [2, KCG, "SQ_INSTS_MFMA", 300.0], [2, KCG, "SQ_LDS_BANK_CONFLICT", 0.0],
            [3, LIB, "SQ_INSTS_MFMA", 50.0], [4, OTHER, "SQ_INSTS_MFMA", 7.0]])
    trace = plr.read_kernel_trace(plr.find_csv([str(tmp_path / "out")], "kernel_trace.csv"))
    assert trace == {KCG: [2000, 1000], LIB: [4000]}
    rows = {r["name"]: r for r in plr.price(trace)}
    fl = 2 * 1024 * 512 * 256
    assert rows[KCG]["gflops"] == [fl / 2000, fl / 1000] and rows[KCG]["min_ns"] == 1000
    assert rows[LIB]["gflops"] == [fl / 4000]              # priced with the generated kernels' shape
    assert plr.price(trace, mnk="2048x512x256")[1]["gflops"] == [2 * fl / 4000]
    ctr = plr.read_counters(plr.find_csv([str(tmp_path / "out")], "counter_collection.csv"))
    assert ctr == {KCG: {"SQ_INSTS_MFMA": 200.0, "SQ_LDS_BANK_CONFLICT": 0.0}, LIB: {"SQ_INSTS_MFMA": 50.0}}
    assert plr.main([str(tmp_path / "out")]) == 0
    text = capsys.readouterr().out
    assert text.splitlines()[0].startswith("eps_torch :  ['%f(Gflops)'" % (fl / 4000))
    assert "eps_kcg :  ['%f(Gflops)', '%f(Gflops)']" % (fl / 2000, fl / 1000) in text
    assert plr.main([str(tmp_path / "out"), "--markdown"]) == 0
    assert "| SQ_INSTS_MFMA | 200 | 50 |" in capsys.readouterr().out
