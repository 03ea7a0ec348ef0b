"""The counter tool's `stamp` step on a hand-made profiler output: scaling by the copy kernel, roles, ratios, and what
bench.py reads back.  CPU only."""
import importlib
import json
import os


def write(path, text):
    os.makedirs(os.path.dirname(path), exist_ok=True)
    with open(path, "w") as f:
        f.write(text)


def test_stamp_scales_by_the_copy_kernel_and_bench_reads_the_ratio(tmp_path):
    counters = importlib.import_module("titanic-flash-41_amd.counters")
    src = str(tmp_path / "raw")
    write(os.path.join(src, "run.json"), json.dumps({"manifest": {"library_sha256": "ab" * 32}, "workloads": ["c2"]}))
    fc1 = "void tf_phase1_stream<8, 8, 4>(StreamArgs, StreamArgs)"
    copy = "tf_probe_copy(unsigned int __vector(4) const*, unsigned int __vector(4)*, unsigned long)"
    write(os.path.join(src, "c2", "trace", "stdout.txt"),
          '{"tiles": 20.0, "active_experts": 20.0, "routes": 24.0, "fc1_algorithmic_bytes": 200000000, "fc2_algorithmic_bytes": 100000000}\n'
          '{"rows": 4, "passes": 64}\n')
    write(os.path.join(src, "c2", "trace", "command.txt"), "rocprofv3 --kernel-trace --stats -- probe\n")
    write(os.path.join(src, "c2", "trace", "w_kernel_stats.csv"),
          '"Name","Calls","TotalDurationNs","AverageNs","Percentage","MinNs","MaxNs","StdDev"\n'
          '"%s",80,3000000,37500.0,50.0,33000,41000,10.0\n"%s",4,400000,100000.0,10.0,99000,101000,1.0\n' % (fc1, copy))
    head = '"Correlation_Id","Dispatch_Id","Kernel_Name","Counter_Name","Counter_Value"\n'
    # the copy kernel moves 256 MiB each way and reads half of that in FETCH_SIZE (KiB), all of it in WRITE_SIZE
    write(os.path.join(src, "c2", "fetch", "w_counter_collection.csv"),
          head + '1,1,"%s","FETCH_SIZE",100000\n2,2,"%s","FETCH_SIZE",102000\n3,3,"%s","FETCH_SIZE",131072\n' % (fc1, fc1, copy))
    write(os.path.join(src, "c2", "write", "w_counter_collection.csv"),
          head + '1,1,"%s","WRITE_SIZE",100\n2,2,"%s","WRITE_SIZE",100\n3,3,"%s","WRITE_SIZE",262144\n' % (fc1, fc1, copy))
    out = str(tmp_path / "counters.json")
    counters.stamp(src, out)
    c = counters.load(out)
    assert c["library_sha256"] == "ab" * 32
    entry = c["workloads"]["c2"]
    assert entry["scale"] == {"fetch": 2.0, "write": 1.0} and entry["tiles"] == 20.0
    rec = entry["kernels"][fc1]
    assert rec["role"] == "fc1" and rec["calls"] == 80 and rec["avg_us"] == 37.5
    want = 101000 * 1024 * 2.0 + 100 * 1024
    assert rec["hbm_bytes"] == want and abs(rec["traffic_over_algorithmic"] - want / 2e8) < 1e-12
    assert counters.traffic_ratio(c, "c2") == rec["traffic_over_algorithmic"]
    assert counters.traffic_ratio(c, "c5") is None and counters.traffic_ratio(None, "c2") is None
    assert entry["kernels"][copy]["role"] == "copy"


def test_stamp_sums_a_projection_that_runs_as_two_kernels(tmp_path):
    counters = importlib.import_module("titanic-flash-41_amd.counters")
    src = str(tmp_path / "raw")
    write(os.path.join(src, "run.json"), json.dumps({"manifest": {"library_sha256": "cd" * 32}, "workloads": ["c5"]}))
    long_units = "void tf_grouped_gemm<0, 256, true>(GemmArgs)"
    last_tiles = "void tf_grouped_gemm<0, 128, true>(GemmArgs)"
    copy = "tf_probe_copy(unsigned int __vector(4) const*, unsigned int __vector(4)*, unsigned long)"
    write(os.path.join(src, "c5", "trace", "stdout.txt"), '{"tiles": 900.0, "fc1_algorithmic_bytes": 3000000000, "fc2_algorithmic_bytes": 2000000000}\n')
    write(os.path.join(src, "c5", "trace", "w_kernel_stats.csv"),
          '"Name","Calls","TotalDurationNs","AverageNs","Percentage","MinNs","MaxNs","StdDev"\n'
          '"%s",6,7200000,1200000.0,50.0,1100000,1300000,10.0\n"%s",6,1800000,300000.0,10.0,290000,310000,1.0\n'
          '"%s",4,400000,100000.0,10.0,99000,101000,1.0\n' % (long_units, last_tiles, copy))
    head = '"Correlation_Id","Dispatch_Id","Kernel_Name","Counter_Name","Counter_Value"\n'
    write(os.path.join(src, "c5", "fetch", "w_counter_collection.csv"),
          head + '1,1,"%s","FETCH_SIZE",1000000\n2,2,"%s","FETCH_SIZE",500000\n3,3,"%s","FETCH_SIZE",131072\n' % (long_units, last_tiles, copy))
    write(os.path.join(src, "c5", "write", "w_counter_collection.csv"),
          head + '1,1,"%s","WRITE_SIZE",100000\n2,2,"%s","WRITE_SIZE",50000\n3,3,"%s","WRITE_SIZE",262144\n' % (long_units, last_tiles, copy))
    out = str(tmp_path / "counters.json")
    counters.stamp(src, out)
    c = counters.load(out)
    role = c["workloads"]["c5"]["roles"]["fc1"]
    want = (1000000 + 500000) * 1024 * 2.0 + (100000 + 50000) * 1024
    assert role["kernels"] == 2 and role["hbm_bytes"] == want and role["avg_us"] == 1500.0
    assert abs(counters.traffic_ratio(c, "c5") - want / 3e9) < 1e-12
    # the kernels keep their own bytes, the ratio belongs to the projection
    assert "traffic_over_algorithmic" not in c["workloads"]["c5"]["kernels"][long_units]
    assert c["workloads"]["c5"]["kernels"][last_tiles]["hbm_bytes"] == 500000 * 1024 * 2.0 + 50000 * 1024
