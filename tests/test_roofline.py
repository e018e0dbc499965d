"""The kernel table of a profiled step: the launches of a step are found in a made-up kernel trace
(other steps and other libraries' kernels around them) and priced with their median times."""
import csv

import pytest

from minivllm_amd.engine import roofline


def write_trace(path, names_and_us):
    t = 1000
    with open(path, "w", newline="") as f:
        w = csv.writer(f)
        w.writerow(["Kind", "Kernel_Name", "Start_Timestamp", "End_Timestamp"])
        for name, us in names_and_us:
            w.writerow(["KERNEL_DISPATCH", name, t, t + int(us * 1000)])
            t += int(us * 1000) + 500


STEP = [("mv_embedding", 100, 0), ("mv_gemm_skinny_norm", 4000, 8000),
        ("mv_attention_decode_fused", 10, 0, 64, 64, 32, 16), ("mv_gemm_skinny", 2000, 4000), ("mv_sample", 300, 600)]


def step_kernels(scale, split=True, rows=8):
    out = [("void embedding_kernel(int const*, void const*)", 1.0 * scale),
           ("void at::native::vectorized_elementwise_kernel<4>(int)", 0.5),
           (f"void gemm_skinny_kernel<{rows}, 1, false, true, __hip_bfloat16>(void*)", 4.0 * scale),
           ("void attention_decode_kernel<128, 4, true, 2>(void*)", 6.0 * scale)]
    if split:
        out.append(("void attention_merge_kernel(float const*)", 2.0 * scale))
    out += [(f"void gemm_skinny_kernel<{rows}, 1, false, false, __hip_bfloat16>(void*)", 3.0 * scale),
            ("void sample_partial_kernel(float const*)", 1.0 * scale), ("void sample_kernel(float const*)", 1.0 * scale)]
    return out


def test_steps_are_found_and_priced(tmp_path):
    trace = [("void add_rmsnorm_kernel<float>(float*)", 9.0), ("Cijk_Alik_Bljk_BBS_BH_MT64x64x32_SN", 50.0)]
    assert roofline.short_name("Custom_Cijk_Alik_Bljk_BBS_BH_Bias_HA_S_SAV_NTD_SK3_UserArgs_MT256x256x64_MI16") == "hipBLASLt BBS MT256x256x64"
    assert roofline._OURS.search("Custom_Cijk_Alik_Bljk_BBS_BH_Bias") and roofline._OURS.search(trace[1][0])
    for scale in (1.0, 1.2, 0.8, 1.0, 5.0):
        trace += step_kernels(scale)
    trace += step_kernels(1.0, rows=4) * 2             # steps of another batch size: other kernels, left out
    trace += [("void embedding_kernel(int const*, void const*)", 1.0)]   # a step that was cut off
    path = str(tmp_path / "x_kernel_trace.csv")
    write_trace(path, trace)
    ledger = roofline.launches(STEP)
    found = roofline.find_windows(roofline.read_trace(path), ledger)
    assert len(found) == 7
    text = roofline.kernel_table(path, ledger, "bfloat16", keys=128, pairs=128, title="t", wall_ms=0.03)
    assert "5 occurrences" in text and "(2 more with other kernels left out)" in text
    line = next(l for l in text.splitlines() if l.startswith("attention_decode_kernel"))
    assert "attention_merge_kernel" in line
    cells = line.split()
    us, kb = float(cells[-9]), float(cells[-6])
    assert us == pytest.approx(8.0) and kb == pytest.approx((10 + 128 * 32) / 1e3, abs=0.06)
    norm_line = next(l for l in text.splitlines() if l.startswith("gemm_skinny_kernel<8,1,false,true"))
    assert float(norm_line.split()[-9]) == pytest.approx(4.0)
    assert "kernels of other libraries inside the step (fills, copies): 1 launches, 0.5 us" in text
    assert "not inside a kernel: 11.5 us" in text       # 30 - 18 - 0.5


def test_one_step_of_a_row_and_errors(tmp_path):
    row = roofline.launches(STEP * 3)
    assert [l.entry for l in roofline.one_step(row)] == [s[0] for s in STEP]
    path = str(tmp_path / "y_kernel_trace.csv")
    write_trace(path, step_kernels(1.0)[:4])
    with pytest.raises(ValueError, match="holds no run of the 5 launches"):
        roofline.kernel_table(path, roofline.launches(STEP), "bfloat16")
    stats = tmp_path / "z_kernel_stats.csv"
    stats.write_text('"Name","Calls","TotalDurationNs"\n"k",1,5\n')
    with pytest.raises(ValueError, match="not a rocprofv3 kernel trace"):
        roofline.read_trace(str(stats))


def test_two_products_of_one_kernel_in_a_row_are_two_launches(tmp_path):
    """A product whose K is split launches its kernel and the one that adds the partial sums; the
    same kernel twice in a row is two products, and only the second kind of kernel may follow within
    a launch."""
    step = [("mv_embedding", 100, 0), ("mv_gemm_tile", 4000, 8000), ("mv_gemm_tile", 2000, 4000),
            ("mv_add_rmsnorm_split", 500, 0), ("mv_gemm_tile", 3000, 6000), ("mv_sample", 300, 600)]
    kernels = [("void embedding_gather_kernel(int const*)", 1.0),
               ("void gemm_tile_kernel<2, 4, true, 3, 2>(TileArgs)", 40.0),
               ("void gemm_tile_kernel<2, 2, false, 4, 2>(TileArgs)", 20.0),
               ("void add_rmsnorm_vec_kernel<bf16, true>(float*)", 5.0),
               ("void gemm_tile_kernel<2, 2, false, 4, 2>(TileArgs)", 15.0),
               ("void gemm_mid_reduce_kernel<bf16>(float const*)", 4.0),
               ("void sample_kernel(float const*)", 2.0)]
    path = str(tmp_path / "t_kernel_trace.csv")
    write_trace(path, kernels * 3)
    found = roofline.find_windows(roofline.read_trace(path), roofline.launches(step))
    assert len(found) == 3
    assert [len(t) for t in found[0].times] == [1, 1, 1, 1, 2, 1]
    text = roofline.kernel_table(path, roofline.launches(step), "bfloat16", title="t")
    assert "3 occurrences" in text
