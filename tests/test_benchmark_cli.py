"""The benchmark-driver counterpart (triton_amd/benchmark.py): record schema and tensor recipe of the reference's
drivers (vanilla_llama_benchmark.py:131-139, :515-547)."""
import json

import pytest

from triton_amd import benchmark


def test_tensor_shapes_follow_the_reference_drivers():
    s = benchmark.tensor_shapes({"M": 16, "N": 4096, "D": 128, "P": 1024})
    assert s["X"] == (16, 4096) and s["WQ"] == (4096, 4096) and s["K_cache"] == (32, 1040, 128)
    assert s["noise"] == (32, 16, 1040) and s["C_out1"] == (32, 1040) and s["O2"] == (16, 4096)
    assert benchmark.tensor_shapes({"M": 16, "N": 4544, "D": 64, "H": 71, "P": 1024})["V_cache"] == (71, 1040, 64)


def test_records_are_appended_like_the_incremental_save(tmp_path):
    out = tmp_path / "r.json"
    rec = {"ir_id": "x", "ir_expression": "y", "execution_time_ms": 1.0, "tensor_config": {"M": 1}, "error": None}
    benchmark.append_record(str(out), rec)
    benchmark.append_record(str(out), dict(rec, ir_id="z"))
    data = json.loads(out.read_text())
    assert [d["ir_id"] for d in data] == ["x", "z"]
    assert set(data[0]) == {"ir_id", "ir_expression", "execution_time_ms", "tensor_config", "error"}


def test_bad_config_file_is_rejected(tmp_path):
    p = tmp_path / "c.json"
    p.write_text(json.dumps([{"M": 16}]))
    with pytest.raises(SystemExit):
        benchmark.main(["--configs", str(p), "--output", str(tmp_path / "o.json")])


@pytest.mark.gpu
@pytest.mark.parametrize("variant", benchmark.VARIANTS)
def test_cli_times_every_variant_and_records_failures(variant, tmp_path):
    import math
    cfgs = tmp_path / "c.json"
    cfgs.write_text(json.dumps([{"M": 16, "N": 512, "D": 64, "H": 8, "P": 40},
                                {"M": 16, "N": 500, "D": 64, "H": 8, "P": 40}]))      # second one is inconsistent
    out = tmp_path / "o.json"
    assert benchmark.main(["--variant", variant, "--configs", str(cfgs), "--output", str(out), "--runs", "5", "--warmup", "2"]) == 0
    data = json.loads(out.read_text())
    assert len(data) == 2
    assert data[0]["error"] is None and 0 < data[0]["execution_time_ms"] < 10 and data[0]["tensor_config"]["N"] == 512
    assert data[1]["error"] and math.isinf(data[1]["execution_time_ms"])


def test_lora_and_gmlp_shapes_follow_their_drivers():
    s = benchmark.tensor_shapes({"M": 16, "N": 1024, "P": 512, "R": 64})
    assert s == {"X": (16, 1024), "W": (1024, 512), "A": (1024, 64), "B": (64, 512), "O": (16, 512)}
    s = benchmark.tensor_shapes({"M": 16, "N": 2048, "K": 1024})
    assert s == {"X": (16, 1024), "W1": (1024, 2048), "W2": (1024, 2048), "O": (16, 2048)}


@pytest.mark.gpu
@pytest.mark.parametrize("variant", benchmark.LINEAR_VARIANTS)
def test_cli_times_lora_and_gmlp_at_the_reference_shapes(variant, tmp_path):
    out = tmp_path / "o.json"
    assert benchmark.main(["--variant", variant, "--output", str(out), "--runs", "5", "--warmup", "2"]) == 0
    data = json.loads(out.read_text())
    assert len(data) == len(benchmark.LORA_CONFIGS if variant == "lora" else benchmark.GMLP_CONFIGS)
    assert all(d["error"] is None and 0 < d["execution_time_ms"] < 10 for d in data)
