"""bench.py's command line: what it must do without a GPU."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _run(*args):
    return subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), *args], capture_output=True, text=True, timeout=300)


def test_more_than_one_gpu_is_refused_with_a_message():
    r = _run("--gpus", "2")
    assert r.returncode == 2
    assert "one GPU only" in r.stderr and r.stdout.strip() == ""


def test_help_names_the_contract_flags():
    r = _run("--help")
    assert r.returncode == 0
    for flag in ("--gpus", "--steps", "--warmup", "--no-cpu-baseline", "--prefill-probe", "--pmc-probe", "--e2e-only"):
        assert flag in r.stdout


def test_per_unit_figures_of_the_workload():
    """The algorithmic bytes the roofline is priced with come from the workload's own shape list: K * N / 4
    per call (the packed matrix of one BitLinear, gpu/pack_weight.py:76-98: four weights per byte), four calls
    per layer at the 2B dimensions of gpu/model.py:41-48 (dim 2560, 20 + 2 * 5 heads of 128, ffn 6912), 30
    layers per step; and the packer really writes that many bytes."""
    import numpy as np

    from bitnet_amd import pack_weight, workload

    dim, heads, kv_heads, head_dim, ffn, layers = 2560, 20, 5, 128, 6912, 30
    want = {"wqkv": (dim, (heads + 2 * kv_heads) * head_dim), "wo": (heads * head_dim, dim), "w13": (dim, 2 * ffn), "w2": (ffn, dim)}
    shapes = workload.shapes_2b()
    assert [sh.name for sh in shapes] == list(want)
    for sh in shapes:
        assert (sh.K, sh.N) == want[sh.name]
        assert sh.weight_bytes == sh.K * sh.N // 4 == workload.packed_bytes(sh.K, sh.N)
        assert sum(sh.parts) == sh.N
    assert workload.N_LAYERS_2B == layers
    per_layer = sum(sh.weight_bytes for sh in shapes)
    assert per_layer == 17367040 and layers * per_layer == 521011200
    # a packed matrix holds exactly K * N / 4 bytes
    import torch

    w = workload.ternary_weight(256, 48, 0)
    assert pack_weight.convert_weight_int8_to_int2(torch.from_numpy(w)).numel() == workload.packed_bytes(256, 48)
    assert set(np.unique(w)) <= {-1, 0, 1}


def test_cpu_baseline_leg_reports_the_harness_protocol():
    """cpu_baseline on a shrunken workload (two small shapes, no GPU): per shape mean and minimum over 200
    timed calls at one thread and at all threads, both thread counts, the build line and the _Nx1 leg."""
    sys.path.insert(0, ROOT)
    import bench
    from bitnet_amd import workload

    small = [workload.LayerShape("a", 0, 256, 64, (64,)), workload.LayerShape("b", 1, 512, 32, (32,))]
    r = bench.cpu_baseline(small, 1, budget_s=0.5)
    assert r["kind"] == "port" and r["unit"] == "GB/s" and r["value"] > 0
    assert r["cores"] == r["threads"]["all"] <= 16 and r["threads"]["single"] == 1 and r["threads"]["host_cpu_count"] >= 1
    assert "march=native" in r["build"] or "mavx2" in r["build"]
    for name in ("a", "b"):
        leg = r["per_shape"][name]
        for key in ("threads_1", f"threads_{r['cores']}"):
            assert leg[key]["iterations"] == 200 and 0 < leg[key]["min_us"] <= leg[key]["mean_us"]
        assert r["M128_Nx1"][name]["iterations"] >= 3 and r["M128_Nx1"][name]["TOPS"] > 0
