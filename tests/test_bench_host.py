"""Host-side pieces of bench.py that need no GPU: the refusal of more than one GPU and the reading of the
profiler's counter files."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)

import bench  # noqa: E402


def test_more_than_one_gpu_is_refused():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert r.returncode != 0 and "one GPU" in r.stderr


def test_counter_file_is_summed_per_phase_and_aggregation(tmp_path):
    rows = ["Correlation_Id,Dispatch_Id,Agent_Id,Queue_Id,Process_Id,Thread_Id,Grid_Size,Kernel_Id,Kernel_Name,"
            "Workgroup_Size,LDS_Block_Size,Scratch_Size,VGPR_Count,Accum_VGPR_Count,SGPR_Count,Counter_Name,Counter_Value,"
            "Start_Timestamp,End_Timestamp"]

    def add(name, grid, counter, value):
        rows.append(f'1,1,0,1,1,1,{grid},1,"{name}",256,0,0,64,0,80,{counter},{value},0,1')

    add("(anonymous namespace)::rof_copy_kernel(HIP_vector_type<float, 4u> const*, HIP_vector_type<float, 4u>*, long)",
        2097152, "FETCH_SIZE", 524288.0)
    add("at::native::some_other_kernel<float, 4, 12, 2, true>()", 64, "FETCH_SIZE", 99.0)
    for _ in range(bench.CHILD_AGGREGATIONS):
        add("void rofk::rof_rows_kernel<float, 4, 12, 5, true>(rofk::AggArgs)", 174080, "FETCH_SIZE", 10.0)      # groups
        add("void rofk::rof_rows_kernel<float, 4, 12, 3, true>(rofk::AggArgs)", 9205760, "FETCH_SIZE", 1000.0)   # segments, streamed
        add("void rofk::rof_rows_kernel<float, 4, 12, 2, true>(rofk::AggArgs)", 36012032, "FETCH_SIZE", 2000.0)  # rows
        add("void rofk::rof_rows_kernel<float, 4, 12, 4, true>(rofk::AggArgs)", 36012032, "FETCH_SIZE", 1000.0)  # rows, more in flight
        add("void rofk::rof_cluster_kernel<unsigned short, 8, 32, 1, false>(rofk::AggArgs)", 4096, "FETCH_SIZE", 500.0)
    path = tmp_path / "rof_counter_collection.csv"
    path.write_text("\n".join(rows) + "\n")
    per, copy = bench.read_counter_csv(str(path))
    assert copy == {"FETCH_SIZE": 524288.0}
    assert per == {("FETCH_SIZE", 0): 1010.0, ("FETCH_SIZE", 1): 3500.0}


def test_offline_figures_cover_the_default_workload():
    t = bench.PROFILED_TRAFFIC[("c4", 3, 47, True)]
    assert set(t["launch"]) == {0, 1} and t["launch"][1]["bytes"] == t["launch"][1]["read_bytes"] + t["launch"][1]["written_bytes"]
    assert t["launch"][1]["bytes"] / 0.94e-3 / 1e9 / bench.HBM_PEAK_GBS < 1.0
