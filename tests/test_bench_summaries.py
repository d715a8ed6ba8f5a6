"""bench.py --summarise on small made-up rocprofv3 CSV files: the text summaries kept under profiles/ come from
this code, so its arithmetic is checked here (no GPU, no rocprofv3)."""
import json
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def run(args, cwd):
    return subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--summarise"] + args, cwd=cwd,
                          stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, check=True).stdout


def test_kernel_trace_summary(tmp_path):
    stats = tmp_path / "stats.csv"
    stats.write_text(
        '"Name","Calls","TotalDurationNs","AverageNs","Percentage","MinNs","MaxNs","StdDev"\n'
        '"void thgpu::gemm_fast_kernel<128, 128, 2, 2, 0, 4, false>(thgpu::GemmArgs)",20,4000000,200000,80.0,1,1,0\n'
        '"thgpu::(anonymous namespace)::pad_planes_kernel(float const*, float*)",10,1000000,100000,20.0,1,1,0\n')
    bench = tmp_path / "bench.json"
    bench.write_text(json.dumps({"roofline": {"flops_per_step": 2e11, "ms_per_step": 1.9, "achieved": 105.0},
                                 "value": 1000.0, "ms_per_step": 2.4}))
    out = run(["kernel-trace", str(stats), str(bench), "2", "--summary-header", "title\\ncommand"], str(tmp_path))
    assert out.startswith("title\ncommand\n")
    # 4 ms of GEMM over 2 steps = 2 ms per step; 2e11 flops / 2 ms = 100 TFLOP/s = 63.6 % of 157.3
    assert "GEMM kernels (10 launches per step): 2.000 ms per step" in out
    assert "100.0 TFLOP/s = 63.6 %" in out and "average GEMM launch 200.0 us" in out
    assert "All kernels: 2.500 ms per step" in out


def test_traffic_summary(tmp_path):
    head = '"Dispatch_Id","Kernel_Name","Counter_Name","Counter_Value"\n'
    fetch, write = tmp_path / "f.csv", tmp_path / "w.csv"
    g = '"void thgpu::gemm_fast_kernel<128, 128, 2, 2, 0, 4, false>(thgpu::GemmArgs)"'
    p = '"thgpu::(anonymous namespace)::pad_planes_kernel(float const*, float*)"'
    fetch.write_text(head + '1,%s,"FETCH_SIZE",51200\n2,%s,"FETCH_SIZE",10240\n' % (g, p))      # KiB, read at half size
    write.write_text(head + '1,%s,"WRITE_SIZE",20480\n2,%s,"WRITE_SIZE",30720\n' % (g, p))
    bench = tmp_path / "bench.json"
    bench.write_text(json.dumps({
        "config": {"workload": "alexnet stack", "batch": 128, "conv_route": "auto", "relu_fused": True},
        "kernels": {"pad_planes": {"gbs": 5000.0, "ms_per_step": 0.01}},
        "gemm_shapes": [{"gemm": "gemm_conv_fwd M=1 J=1 R=1 tile=128x128 split=1"}]}))
    out = run(["traffic", str(fetch), str(write), str(bench), "1"], str(tmp_path))
    # GEMM: 51200 KiB * 2 / 1024 = 100 MiB fetched, 20 MiB written
    assert "GEMM family: 120.0 MiB per step over 1 launches = 120.0 MiB" in out
    check = json.loads(out.split("bench_check: ")[1])
    assert check["gemm_bytes_per_launch"] == 120 * 1048576 and check["route"] == "auto" and check["fused"] is True
    pad = [l for l in out.splitlines() if l.startswith("pad_planes")][0].split()
    assert float(pad[2]) == 20.0 and float(pad[3]) == 30.0 and float(pad[4]) == 50.0      # fetch, write, total MiB
