"""Benchmark driver (YAML shape list -> CSV): column set and flags of the reference's
benchmarks/tritonblas_matmul.py; shape lists of datasets/generate_grid*.py."""
import csv

import pytest
import torch
import yaml

REFERENCE_COLUMNS = ["m", "n", "k", "mnk", "macro_tile", "bytes", "flops", "tritonblas_gflops", "a_type", "b_type", "c_type",
                     "d_type", "compute_type", "in_dtype", "out_dtype", "init_type", "transA", "transB", "us", "alpha", "beta",
                     "mode"]   # benchmarks/tritonblas_matmul.py:287-293


def test_csv_columns_are_the_reference_ones():
    from tritonblas_amd.benchmarks import matmul_bench
    assert matmul_bench.FIELDNAMES == REFERENCE_COLUMNS


def test_generate_grid_presets(tmp_path):
    from tritonblas_amd.benchmarks import generate_grid
    out = tmp_path / "g.yaml"
    generate_grid.main(["--preset", "grid", "--min", "1024", "--max", "2048", "--step", "1024", "-o", str(out)])
    cases = yaml.safe_load(out.read_text())
    assert len(cases) == 8 and cases[0] == {"m": 1024, "n": 1024, "k": 1024, "in_dtype": "float16", "out_dtype": "float16",
                                            "transA": "T", "transB": "N"}
    generate_grid.main(["--preset", "fp4", "--out-dtype", "bfloat16", "-o", str(out)])
    cases = yaml.safe_load(out.read_text())
    assert len(cases) == 19 and all(c["in_dtype"] == "fp4" and c["k"] % 32 == 0 for c in cases)   # generate_grid_fp4.py:12-36
    assert (cases[0]["m"], cases[0]["n"], cases[0]["k"]) == (256, 2048, 8192)


def test_dtype_names():
    import torch
    from tritonblas_amd.benchmarks.matmul_bench import str_to_dtype
    assert str_to_dtype("bfloat16") is torch.bfloat16 and str_to_dtype("torch.float8_e4m3fn") is torch.float8_e4m3fn
    assert str_to_dtype("fp4") == "fp4"
    assert str_to_dtype("int8") is torch.int8 and str_to_dtype("float32") is torch.float32
    with pytest.raises(ValueError):
        str_to_dtype("float64")


@pytest.mark.gpu
@pytest.mark.parametrize("flags", [[], ["--enable-streamk"], ["--work-stealing"]])
def test_driver_runs_a_shape_list_with_correctness_check(tmp_path, flags):
    from tritonblas_amd.benchmarks import matmul_bench
    print(f"bench driver {flags}", flush=True)
    cases = [
        {"m": 256, "n": 512, "k": 1024, "in_dtype": "bfloat16", "out_dtype": "bfloat16", "transA": "T", "transB": "N"},
        {"m": 300, "n": 200, "k": 512, "in_dtype": "float16", "out_dtype": "float16", "transA": "T", "transB": "T"},
        {"m": 512, "n": 256, "k": 2048, "in_dtype": "float8_e4m3fn", "out_dtype": "bfloat16", "transA": "T", "transB": "N"},
        {"m": 256, "n": 512, "k": 1024, "in_dtype": "float8_e5m2", "out_dtype": "bfloat16", "transA": "T", "transB": "N"},
        {"m": 384, "n": 256, "k": 1024, "in_dtype": "int8", "out_dtype": "bfloat16", "transA": "T", "transB": "N"},
        {"m": 256, "n": 384, "k": 512, "in_dtype": "int8", "out_dtype": "int8", "transA": "T", "transB": "N"},
        {"m": 320, "n": 256, "k": 768, "in_dtype": "float32", "out_dtype": "float32", "transA": "T", "transB": "T"},
    ]
    if not flags:
        cases.append({"m": 128, "n": 256, "k": 1024, "in_dtype": "fp4", "out_dtype": "bfloat16", "transA": "T", "transB": "N"})
    src, dst = tmp_path / "shapes.yaml", tmp_path / "out.csv"
    src.write_text(yaml.safe_dump(cases))
    matmul_bench.main(["--input-yaml", str(src), "--output-csv", str(dst), "--checkcorrectness", "--n-warmup", "2",
                       "--n-repeat", "3"] + flags)
    rows = list(csv.DictReader(dst.open()))
    assert len(rows) == len(cases) and list(rows[0].keys()) == REFERENCE_COLUMNS
    want_mode = "work_stealing" if "--work-stealing" in flags else ("streamk" if "--enable-streamk" in flags else "persistent")
    assert all(r["mode"] == want_mode and float(r["tritonblas_gflops"]) > 0 for r in rows)


def test_cu_sweep_steps():
    from tritonblas_amd.benchmarks.matmul_bench import cu_sweep_steps, _fieldnames
    assert cu_sweep_steps(256, 8, 32, 3) == [256, 248, 240, 232]
    assert cu_sweep_steps(304, 8, 38, 34) == [304 - 8 * r for r in range(35)]          # the reference's MI300X default
    assert cu_sweep_steps(256, 8, 32, 100)[-1] == 8                                    # at least one CU per XCD stays
    assert _fieldnames([{"active_cus": 8, "m": 1}]) == ["active_cus"] + REFERENCE_COLUMNS
    assert _fieldnames([{"m": 1}]) == REFERENCE_COLUMNS and _fieldnames([]) == REFERENCE_COLUMNS


def test_masked_cu_sweep_parent(tmp_path, monkeypatch):
    """--cu-sweep --cu-mask (reference benchmarks/tritonblas_matmul.py:381-412): the parent asks a child for the CU
    counts, then runs one child per step with the balanced ROC_GLOBAL_CU_MASK of that step and without the sweep /
    output flags, and concatenates their JSON rows.  The children are faked here; the parent must not touch a GPU."""
    import json
    from types import SimpleNamespace
    from tritonblas_amd.benchmarks import matmul_bench
    from tritonblas_amd.benchmarks.common import build_balanced_hex_mask
    calls = []

    def fake_child(argv_tail, env=None):
        calls.append((list(argv_tail), None if env is None else env.get("ROC_GLOBAL_CU_MASK")))
        if "--_cu-info" in argv_tail:
            return SimpleNamespace(returncode=0, stdout="[256, 8, 32]\n", stderr="")
        active = int(argv_tail[argv_tail.index("--_active-cus") + 1])
        return SimpleNamespace(returncode=0, stdout="noise\n" + json.dumps([{"active_cus": active, "m": 1}]) + "\n", stderr="")

    monkeypatch.setattr(matmul_bench, "_child", fake_child)
    monkeypatch.setattr(torch.cuda, "current_device", lambda: (_ for _ in ()).throw(AssertionError("GPU call in the parent")))
    dst = tmp_path / "out.csv"
    matmul_bench.main(["--input-yaml", "shapes.yaml", "--output-csv", str(dst), "--work-stealing", "--cu-sweep", "--cu-mask",
                       "--cu-sweep-max-remove", "2", "--n-repeat", "3"])
    assert calls[0][0] == ["--input-yaml", "shapes.yaml", "--_cu-info"]
    assert [c[1] for c in calls[1:]] == [None, build_balanced_hex_mask(1, 8, 32), build_balanced_hex_mask(2, 8, 32)]
    for argv_tail, _ in calls[1:]:
        assert argv_tail[:5] == ["--input-yaml", "shapes.yaml", "--work-stealing", "--n-repeat", "3"]
        assert "--cu-sweep" not in argv_tail and "--cu-mask" not in argv_tail and "--output-csv" not in argv_tail
    rows = list(csv.DictReader(dst.open()))
    assert [int(r["active_cus"]) for r in rows] == [256, 248, 240]


@pytest.mark.gpu
@pytest.mark.parametrize("flags", [["--work-stealing"], ["--work-stealing", "--global-atomic"], ["--work-stealing", "--hierarchical"], []])
def test_driver_cu_sweep(tmp_path, flags):
    from tritonblas_amd.benchmarks import matmul_bench
    from tritonblas_amd.benchmarks.common import get_cu_info
    print(f"bench driver cu sweep {flags}", flush=True)
    cases = [
        {"m": 1024, "n": 1024, "k": 512, "in_dtype": "bfloat16", "out_dtype": "bfloat16", "transA": "T", "transB": "N"},
        {"m": 512, "n": 768, "k": 1024, "in_dtype": "float8_e4m3fn", "out_dtype": "bfloat16", "transA": "T", "transB": "N"},
    ]
    src, dst = tmp_path / "shapes.yaml", tmp_path / "out.csv"
    src.write_text(yaml.safe_dump(cases))
    matmul_bench.main(["--input-yaml", str(src), "--output-csv", str(dst), "--checkcorrectness", "--n-warmup", "1",
                       "--n-repeat", "2", "--cu-sweep", "--cu-sweep-max-remove", "2"] + flags)
    rows = list(csv.DictReader(dst.open()))
    full, xcds, _ = get_cu_info(0)
    assert list(rows[0].keys()) == ["active_cus"] + REFERENCE_COLUMNS
    assert [int(r["active_cus"]) for r in rows] == [full] * 2 + [full - xcds] * 2 + [full - 2 * xcds] * 2
