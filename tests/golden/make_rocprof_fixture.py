"""Writes tests/golden/rocprof/: two tiny rocprofv3 output trees in the column layout rocprofv3 7.2 writes
(<pass>_kernel_trace.csv, <pass>_counter_collection.csv, <pass>.stdout), with round numbers, for
tests/test_profiles_summary.py.  The numbers are chosen so that every figure of the summary is known by construction:

bench case (gemm_x16_f16_8192): 12 dispatches of the GEMM kernel; the first 7 take 900 us (unsettled chip), the timed
last 5 take 700, 710, 720, 730, 740 us back to back -> median 720 us.  Counter passes: every dispatch 800 us,
GRBM_GUI_ACTIVE = 8 XCDs x 2.0 GHz x 800 us = 1.28e7, SQ_VALU_MFMA_BUSY_CYCLES = 0.75 x 1024 SIMDs x 1.6e6 cycles;
TCC hits 3 : misses 1; FETCH_SIZE 400,000 KiB with a calibration kernel that read 128 MiB and counted 65,536 KiB
(factor 2); WRITE_SIZE 150,000 KiB, calibration 131,072 KiB (factor 1).

shapes case (skinny_cfg4 with two shapes): shape 1 runs split-K (GEMM 10 us + reduction 2 us, 3 us after it), shape 2
one kernel of 20 us; 6 calls each of which the last 4 are timed.

    python tests/golden/make_rocprof_fixture.py
"""
import csv
import json
import os

HERE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "rocprof")
TRACE_COLS = ["Kind", "Agent_Id", "Queue_Id", "Stream_Id", "Thread_Id", "Dispatch_Id", "Kernel_Id", "Kernel_Name", "Correlation_Id",
              "Start_Timestamp", "End_Timestamp", "LDS_Block_Size", "Scratch_Size", "VGPR_Count", "Accum_VGPR_Count", "SGPR_Count",
              "Workgroup_Size_X", "Workgroup_Size_Y", "Workgroup_Size_Z", "Grid_Size_X", "Grid_Size_Y", "Grid_Size_Z"]
PMC_COLS = ["Correlation_Id", "Dispatch_Id", "Agent_Id", "Queue_Id", "Process_Id", "Thread_Id", "Grid_Size", "Kernel_Id", "Kernel_Name",
            "Workgroup_Size", "LDS_Block_Size", "Scratch_Size", "VGPR_Count", "Accum_VGPR_Count", "SGPR_Count", "Counter_Name",
            "Counter_Value", "Start_Timestamp", "End_Timestamp"]
GEMM = "_ZN4mmbo15gemm_x16_kernelIDF16_Lb0ELb0ELi256ELi256ELi2ELi2ELi5ELb1ELi1EEEvNS_8GemmArgsE"
RING = "_ZN4mmbo16gemm_ring_kernelIDF16_Lb0ELb0ELi64ELi64ELi2ELi2ELi6EEEvNS_8GemmArgsE"
RING32 = "void mmbo::gemm_ring_kernel<float, false, false, 64, 64, 2, 2, 6>(mmbo::GemmArgs)"
REDUCE = "_ZN4mmbo20splitk_reduce_kernelIDF16_Lb1EEEvNS_8GemmArgsE"
FILL = "void at::native::(anonymous namespace)::distribution_elementwise_grid_stride_kernel<float, 4>(long)"
CALIB = "void at::native::vectorized_elementwise_kernel<8, at::native::CUDAFunctor_add<c10::Half>, std::array<char*, 2ul> >(int)"
PROBE = "mmbo::probe_mfma_kernel<1>(float*)"


def write_trace(path, dispatches):
    os.makedirs(os.path.dirname(path), exist_ok=True)
    with open(path, "w", newline="") as f:
        w = csv.writer(f, quoting=csv.QUOTE_NONNUMERIC)
        w.writerow(TRACE_COLS)
        for i, (name, start, end) in enumerate(dispatches, 1):
            w.writerow(["KERNEL_DISPATCH", "Agent 1", 1, 0, 469, i, 8, name, i, start, end, 0, 0, 128, 256, 96, 256, 1, 1, 65536, 1, 1])


def write_counters(path, dispatches, values):
    """values(name, index among the dispatches) -> {counter: value}"""
    os.makedirs(os.path.dirname(path), exist_ok=True)
    with open(path, "w", newline="") as f:
        w = csv.writer(f, quoting=csv.QUOTE_NONNUMERIC)
        w.writerow(PMC_COLS)
        for i, (name, start, end) in enumerate(dispatches, 1):
            for cname, v in values(name, i).items():
                w.writerow([i, i, "Agent 1", 1, 515, 515, 65536, 13, name, 256, 0, 0, 128, 256, 96, cname, f"{v:.6f}", start, end])


def bench_case():
    root = os.path.join(HERE, "bench_f16")
    t = 1_000_000_000
    disp = [(FILL, t, t + 90_000), (CALIB, t + 100_000, t + 160_000)]
    t += 200_000
    for d in [900_000] * 7 + [700_000, 710_000, 720_000, 730_000, 740_000]:
        disp.append((GEMM, t, t + d))
        t += d                                   # back to back: gap 0
    disp.append((PROBE, t + 50_000, t + 60_050_000))
    write_trace(os.path.join(root, "trace", "trace_kernel_trace.csv"), disp)
    rec = {"metric": "GEMM TFLOP/s + % of MFMA peak, fp16 & fp32 at 8192^3, 1 MI355X", "value": 1520.0, "unit": "TFLOP/s", "steps": 5,
           "warmup": 2, "ms_per_step": 0.7234, "dtype": "f16",
           "config": {"workload": "HGEMM NN M=N=K=8192", "tile_config": "MT256x256x32_WT128x128_W4_GSU01_DTL1_RING5_MFMA16x16x32_ACC"},
           "roofline": {"frac": 0.608},
           "mfma_issue_ceiling": {"f16_random_operands": {"tflops": 1900.0, "shader_mhz": 1900},
                                  "f16_ones_operands": {"tflops": 2400.0, "shader_mhz": 2400}}}
    for p in ("trace", "sq", "tcc", "fetch", "write"):
        with open(os.path.join(root, p + ".stdout"), "w") as f:
            f.write("some log line that is not JSON\n" + json.dumps(rec) + "\n")
    # counter passes: 2 other kernels, then 10 GEMM dispatches of 800 us (the first tenth = 1 dispatch is dropped: give it odd values)
    t = 2_000_000_000
    pd = [(FILL, t, t + 90_000), (CALIB, t + 100_000, t + 160_000)]
    t += 200_000
    for _ in range(10):
        pd.append((GEMM, t, t + 800_000))
        t += 805_000
    first_gemm = 3

    def sq(name, i):
        if name != GEMM:
            return {"GRBM_GUI_ACTIVE": 1000.0, "SQ_VALU_MFMA_BUSY_CYCLES": 0.0}
        odd = 3.0 if i == first_gemm else 1.0
        return {"GRBM_GUI_ACTIVE": 1.28e7 * odd, "SQ_VALU_MFMA_BUSY_CYCLES": 0.75 * 1024 * 1.6e6, "SQ_LDS_BANK_CONFLICT": 0.0,
                "SQ_LDS_IDX_ACTIVE": 5.0e7, "SQ_INSTS_VALU_MFMA_MOPS_F16": 2147483648.0, "SQ_INSTS_VALU_MFMA_MOPS_F32": 0.0}

    def tcc(name, i):
        return {"TCC_HIT_sum": 6.0e7, "TCC_MISS_sum": 2.0e7} if name == GEMM else {"TCC_HIT_sum": 1.0, "TCC_MISS_sum": 1.0}

    def fetch(name, i):
        return {"FETCH_SIZE": 400_000.0 if name == GEMM else 65_536.0 if name == CALIB else 10.0}

    def write(name, i):
        return {"WRITE_SIZE": 150_000.0 if name == GEMM else 131_072.0 if name == CALIB else 262_144.0}

    for p, fn in (("sq", sq), ("tcc", tcc), ("fetch", fetch), ("write", write)):
        write_trace(os.path.join(root, p, p + "_kernel_trace.csv"), pd)
        write_counters(os.path.join(root, p, p + "_counter_collection.csv"), pd, fn)


def shapes_case():
    root = os.path.join(HERE, "shapes")
    recs = []
    t = 5_000_000_000
    disp = [(FILL, t, t + 5_000)]
    t += 10_000
    for _ in range(6):                            # shape 1: split-K, GEMM 10 us, reduction 2 us starting 3 us later
        disp += [(RING, t, t + 10_000), (REDUCE, t + 13_000, t + 15_000)]
        t += 18_000                               # the next GEMM starts 3 us after the reduction ends
    disp.append((FILL, t, t + 5_000))
    t += 10_000
    for _ in range(6):                            # shape 2: one kernel of 20 us, back to back
        disp.append((RING32, t, t + 20_000))
        t += 20_000
    disp.append((PROBE, t + 50_000, t + 60_050_000))
    base = {"batch": 1, "transA": "N", "transB": "N", "alpha": 1.0, "beta": 0.0, "calls_total": 6, "calls_timed": 4}
    recs.append(dict(base, spec="h,N,N,4096,128,4096,1,1,0", dtype="h", m=4096, n=128, k=4096, config="MT064x064x32_GSU02",
                     algorithmic_bytes=(4096 * 4096 + 4096 * 128 + 4096 * 128) * 2, gpu_ms_median=0.0155, tflops=277.1,
                     frac_of_peak=0.1108, bound="hbm"))
    recs.append(dict(base, spec="s,N,N,1024,1024,1024,1,1,0", dtype="s", m=1024, n=1024, k=1024, config="MT064x064x16_GSU01",
                     algorithmic_bytes=3 * 1024 * 1024 * 4, gpu_ms_median=0.0201, tflops=106.8, frac_of_peak=0.679, bound="mfma"))
    ceil = {"mfma_issue_ceiling": {"f32_random_operands": {"tflops": 150.0, "shader_mhz": 2300},
                                   "f16_random_operands": {"tflops": 1900.0, "shader_mhz": 1900}}}
    for p in ("trace", "sq", "fetch", "write"):
        write_trace(os.path.join(root, p, p + "_kernel_trace.csv"), disp)
        # (a counter pass sizes its groups by itself: here it times the last 2 of its 6 calls per shape, the trace pass 4)
        mine = recs if p == "trace" else [dict(r, calls_timed=2) for r in recs]
        with open(os.path.join(root, p + ".stdout"), "w") as f:
            f.write("\n".join(json.dumps(r) for r in mine) + "\n" + json.dumps(ceil) + "\n")

    def sq(name, i):
        # short kernels: busy relative to the duration at 2.4 GHz; 10 us x 2.4 GHz = 24,000 cycles, a quarter of them busy
        return {"GRBM_GUI_ACTIVE": 5.0e5, "SQ_VALU_MFMA_BUSY_CYCLES": (0.25 * 24_000 if name == RING else 0.5 * 48_000) * 1024,
                "SQ_LDS_BANK_CONFLICT": 0.0, "SQ_LDS_IDX_ACTIVE": 1.0e5}

    write_counters(os.path.join(root, "sq", "sq_counter_collection.csv"), disp, sq)
    write_counters(os.path.join(root, "fetch", "fetch_counter_collection.csv"), disp,
                   lambda name, i: {"FETCH_SIZE": 20_000.0 if name == RING else 1_000.0 if name == REDUCE else 6_000.0})
    write_counters(os.path.join(root, "write", "write_counter_collection.csv"), disp,
                   lambda name, i: {"WRITE_SIZE": 2_000.0 if name == RING else 1_000.0 if name == REDUCE else 4_096.0})


if __name__ == "__main__":
    bench_case()
    shapes_case()
    print("wrote", HERE)
