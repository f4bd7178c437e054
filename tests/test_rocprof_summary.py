"""The rocprofv3 summary helper (sddmm_gpu_amd/rocprof.py) on hand-written CSV files of known content: the
copy-probe scaling of FETCH_SIZE / WRITE_SIZE, bytes per step, LDS conflicts per active cycle, kernel
durations taken from the pass without counters, and the text form that bench.py reads back."""
import csv
import json
import os

from sddmm_gpu_amd import rocprof

TILE = "void (anonymous namespace)::sddmm_tile_kernel<8, 4, 0, 12, false, false>(sddmm::TileArgs)"
GATHER = "void (anonymous namespace)::sddmm_tile_kernel<8, 4, 0, 4, true, false>(sddmm::TileArgs)"
PROBE = "(anonymous namespace)::sddmm_copy_probe_kernel(HIP_vector_type<float, 4u> const*, HIP_vector_type<float, 4u>*, long)"
OTHER = "void at::native::vectorized_elementwise_kernel<4, FillFunctor<float> >(int)"
VALUES = "sddmm::gather_values_kernel(int const*, float const*, float*, long)"


def write_pass(d, counters, durations, run):
    os.makedirs(d, exist_ok=True)
    if counters:
        with open(os.path.join(d, "p_counter_collection.csv"), "w", newline="") as f:
            w = csv.writer(f, quoting=csv.QUOTE_NONNUMERIC)
            w.writerow(["Correlation_Id", "Dispatch_Id", "Agent_Id", "Queue_Id", "Process_Id", "Thread_Id", "Grid_Size", "Kernel_Id",
                        "Kernel_Name", "Workgroup_Size", "LDS_Block_Size", "Scratch_Size", "VGPR_Count", "Accum_VGPR_Count", "SGPR_Count",
                        "Counter_Name", "Counter_Value", "Start_Timestamp", "End_Timestamp"])
            for disp, (kernel, name, value) in enumerate(counters, 1):
                # one row per (dispatch, counter, die): the helper must add the dies up
                for part in (0.25, 0.75):
                    w.writerow([disp, disp, "Agent 1", 1, 1, 1, 1024, 7, kernel, 256, 0, 0, 64, 0, 32, name, value * part, 0, 1])
    with open(os.path.join(d, "p_kernel_trace.csv"), "w", newline="") as f:
        w = csv.writer(f, quoting=csv.QUOTE_NONNUMERIC)
        w.writerow(["Kind", "Agent_Id", "Queue_Id", "Stream_Id", "Thread_Id", "Dispatch_Id", "Kernel_Id", "Kernel_Name", "Correlation_Id",
                    "Start_Timestamp", "End_Timestamp"])
        for disp, (kernel, ns) in enumerate(durations, 1):
            w.writerow(["KERNEL_DISPATCH", "Agent 1", 1, 0, 1, disp, 7, kernel, disp, 1000, 1000 + ns])
    with open(os.path.join(d, "run.json"), "w") as f:
        f.write("some warning line\n" + json.dumps(run) + "\n")


def test_summary_scales_by_the_copy_probe(tmp_path):
    run = {"config": {"executes": 2, "argv": ["--no-cpu", "--copy-probe"]}, "copy_probe_bytes_each_way": 1 << 20}
    # the probe moves 1 MiB = 1024 KiB each way; FETCH_SIZE reads 512 for it (factor 2), WRITE_SIZE 1024 (factor 1)
    write_pass(tmp_path / "fetch", [(TILE, "FETCH_SIZE", 100.0), (GATHER, "FETCH_SIZE", 10.0), (TILE, "FETCH_SIZE", 300.0),
                                    (GATHER, "FETCH_SIZE", 30.0), (PROBE, "FETCH_SIZE", 512.0), (OTHER, "FETCH_SIZE", 999.0),
                                    (VALUES, "FETCH_SIZE", 50.0)],
               [(TILE, 900_000), (GATHER, 300_000)], run)
    write_pass(tmp_path / "write", [(TILE, "WRITE_SIZE", 40.0), (TILE, "WRITE_SIZE", 40.0), (GATHER, "WRITE_SIZE", 4.0),
                                    (GATHER, "WRITE_SIZE", 4.0), (PROBE, "WRITE_SIZE", 1024.0)],
               [(TILE, 800_000), (GATHER, 250_000)], run)
    write_pass(tmp_path / "lds", [(TILE, "SQ_LDS_BANK_CONFLICT", 50.0), (TILE, "SQ_LDS_IDX_ACTIVE", 1000.0), (TILE, "SQ_INSTS_VALU", 160.0),
                                  (TILE, "SQ_INSTS_VALU_FMA_F32", 128.0)],
               [(TILE, 950_000)], run)
    write_pass(tmp_path / "stats", [], [(TILE, 640_000), (TILE, 660_000), (GATHER, 200_000), (GATHER, 200_000), (PROBE, 5)],
               {"config": {"executes": 2, "argv": ["--no-cpu"]}})
    s = rocprof.summarize(str(tmp_path))
    # fetch: (100 + 300 + 10 + 30) KiB x 1024 x 2 / 2 steps; the fill kernel and the value re-ordering are not part of a step
    assert s["hbm"]["FETCH_SIZE"]["scale_factor"] == 2.0 and s["hbm"]["FETCH_SIZE"]["bytes_per_step"] == 440 * 1024
    assert s["hbm"]["WRITE_SIZE"]["scale_factor"] == 1.0 and s["hbm"]["WRITE_SIZE"]["bytes_per_step"] == 44 * 1024
    assert s["traffic"] == 484 * 1024
    assert s["hbm"]["FETCH_SIZE"]["by_kernel"]["sddmm_tile_kernel<8,4,0,12,false,false>"] == 400 * 1024
    tile = s["kernels"]["sddmm_tile_kernel<8,4,0,12,false,false>"]
    assert tile["lds_bank_conflict_per_active"] == 0.05 and tile["fma_share_of_valu"] == 0.8
    assert tile["avg_us"] == 650.0            # from the pass without counters, not from the slower counter passes
    assert s["kernels"]["sddmm_tile_kernel<8,4,0,4,true,false>"]["avg_us"] == 200.0
    assert s["lds_bank_conflict_per_active"] == 0.05
    text = rocprof.as_text(s)
    assert "rocprofv3 --pmc FETCH_SIZE --kernel-trace" in text and "python3 bench.py --no-cpu --copy-probe" in text
    assert "rocprofv3 --stats --kernel-trace" in text
    p = tmp_path / "summary.txt"
    p.write_text(text)
    assert rocprof.traffic_from_profile_text(str(p)) == 484 * 1024
    assert rocprof.traffic_from_profile_text(str(tmp_path / "none.txt")) is None


def test_counters_without_a_probe_are_not_scaled(tmp_path):
    write_pass(tmp_path / "fetch", [(TILE, "FETCH_SIZE", 100.0)], [(TILE, 1000)], {"config": {"executes": 1}})
    s = rocprof.summarize(str(tmp_path))
    assert s["traffic"] is None and any("not scaled" in n for n in s["notes"])
    assert rocprof.short_name(TILE) == "sddmm_tile_kernel<8,4,0,12,false,false>"
    assert rocprof.is_step_kernel(TILE) and not rocprof.is_step_kernel(PROBE) and not rocprof.is_step_kernel(VALUES)


def test_committed_profiles_hold_the_traffic_line():
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    for name, lo, hi in (("hbm_traffic_config3_k128_auto.txt", 1.4e9, 6e9), ("hbm_traffic_config4_k64_auto.txt", 4e9, 6e10)):
        t = rocprof.traffic_from_profile_text(os.path.join(root, "profiles", name))
        assert t is not None and lo < t < hi, (name, t)
