"""i_amd.profile: the per-kernel report over a rocprofv3 (rocpd SQLite) result file."""
import sqlite3

from i_amd import profile


def make_db(path, with_counters):
    db = sqlite3.connect(path)
    db.execute("create table kernels (name text, start integer, end integer, duration integer, vgpr_count integer, "
               "lds_size integer, workgroup_x integer)")
    rows = [("attn_fwd_bf16_d128_bn64_direct_w8", 10, 2_000_000, 512), ("attn_fwd_bf16_d128_bn64_direct_w8", 30, 1_800_000, 512),
            ("row_softmax_wave_v16", 20, 90_000, 256), ("f0", 40, 5_000, 64), ("f2_gw", 50, 7_000, 64),
            ("void at::native::vectorized_elementwise_kernel<4>(int)", 60, 3_000, 256)]
    for name, start, dur, wg in rows:
        db.execute("insert into kernels values (?, ?, ?, ?, ?, ?, ?)", (name, start, start + dur, dur, 246, 65536, wg))
    if with_counters:
        db.execute("create table counters_collection (kernel_name text, counter_name text, value real)")
        for v in (100.0, 300.0):
            db.execute("insert into counters_collection values ('row_softmax_wave_v16', 'FETCH_SIZE', ?)", (v,))
        db.execute("insert into counters_collection values ('void at::native::copy(int)', 'FETCH_SIZE', 7.0)")
    db.commit()
    db.close()


def test_kernel_rows_are_grouped_sorted_and_filtered(tmp_path):
    path = str(tmp_path / "run_results.db")
    make_db(path, with_counters=False)
    rows = profile.kernel_rows(path)
    assert [r.name for r in rows][:2] == ["attn_fwd_bf16_d128_bn64_direct_w8", "row_softmax_wave_v16"]
    attn = rows[0]
    assert attn.calls == 2 and abs(attn.avg_us - 1900.0) < 1e-9 and attn.min_us == 1800.0 and attn.max_us == 2000.0
    assert abs(sum(r.share for r in rows) - 1.0) < 1e-12
    ours = profile.kernel_rows(path, ours_only=True)
    assert {r.name for r in ours} == {"attn_fwd_bf16_d128_bn64_direct_w8", "row_softmax_wave_v16", "f0", "f2_gw"}
    assert profile.dispatch_durations_us(path, "attn_fwd_bf16_d128_bn64_direct_w8") == [2000.0, 1800.0]
    assert profile.counter_rows(path) == []
    text = profile.format_report(path, ours_only=True)
    assert "| attn_fwd_bf16_d128_bn64_direct_w8 | 2 | 1900.0 | 1800.0 | 2000.0 |" in text and "vectorized" not in text


def test_counters_are_averaged_per_kernel(tmp_path):
    path = str(tmp_path / "pmc_results.db")
    make_db(path, with_counters=True)
    rows = profile.counter_rows(path, ours_only=True)
    assert len(rows) == 1
    c = rows[0]
    assert (c.kernel, c.counter, c.dispatches, c.avg, c.min, c.max) == ("row_softmax_wave_v16", "FETCH_SIZE", 2, 200.0, 100.0, 300.0)
    assert "| row_softmax_wave_v16 | FETCH_SIZE | 2 | 200 | 100 | 300 |" in profile.format_report(path)


def test_names_of_this_backend():
    """Every name the backend can launch is counted as its own: every extern "C" kernel of the code object's source,
    the second-pass kernels of the split loops among them, and the generated kernels in all their forms."""
    import re
    from pathlib import Path

    kernels = Path(profile.__file__).resolve().parent / "csrc" / "kernels"
    source = "".join(p.read_text() for p in sorted(kernels.glob("*")) if p.suffix in (".hip", ".h"))
    # names spelled out, and the ones macros put together (checked by a representative of each family below)
    spelled = set(re.findall(r'extern "C" __global__ void (?:__launch_bounds__\([^)]*\) )?(\w+)\(', source))
    spelled = {n for n in spelled if "##" not in n and not n.endswith("_")}
    assert {"splitk_reduce", "attn_kv_merge", "pad_rows_b16", "pad_rows_b32", "transpose_b32", "shader_clock_probe"} <= spelled
    for name in sorted(spelled):
        assert profile.is_backend_kernel(name), name
    for name in ("attn_fwd_f32_d64_bn32", "attn_fwd_bf16_d128_bn64_direct_w8_f32scale_pad", "gemm_nn_bf16_256x256x64_direct",
                 "gemm_nt_f32_128x128x32_direct", "row_norm_block", "row_exp_wave_s4", "row_scaled_softmax_parts_apply_v", "transpose_b16",
                 "convert_f32_to_bf16", "f0", "f12_w", "f3_g", "f3_gw", "ilang_fill", "ilang_combine", "ilang_combine_w"):
        assert profile.is_backend_kernel(name), name
    for name in ("void at::native::vectorized_elementwise_kernel<4>(int)", "__amd_rocclr_copyBuffer", "foo", "f0x", "f1_p2"):
        assert not profile.is_backend_kernel(name), name
