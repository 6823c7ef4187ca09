"""The evaluation-CLI counterpart (triton_amd/evaluate.py): flags and model constants of the reference's
convert_eval_rms.py (:11-16, :33-60); on the GPU, every variant at both models against eager PyTorch."""
import json

import pytest

from triton_amd import evaluate


def test_model_constants_are_the_reference_ones():
    assert evaluate.constants("llama") == {"M": 16, "D": 128, "N": 4096, "P": 1024, "H": 32}
    assert evaluate.constants("falcon") == {"M": 16, "D": 64, "N": 4544, "P": 1024, "H": 71}
    with pytest.raises(ValueError):
        evaluate.constants("gpt")


def test_convert_only_prints_the_module_interface(capsys):
    assert evaluate.main(["--n", "7", "--m", "falcon", "--t", "keyformer"]) == 0
    out = capsys.readouterr().out
    assert "[Case7]" in out and "'noise'" in out and "BLOCK_PARAMS = []" in out


@pytest.mark.parametrize("argv", (["--t", "mlp"], ["--m", "gpt"], ["--o", "3"]))
def test_bad_flags_are_rejected(argv):
    with pytest.raises(SystemExit):
        evaluate.main(argv)


@pytest.mark.gpu
@pytest.mark.parametrize("model", ("llama", "falcon"))
@pytest.mark.parametrize("variant", evaluate.VARIANTS)
def test_every_variant_matches_eager_pytorch_on_the_reference_inputs(variant, model, tmp_path, monkeypatch):
    import functools
    monkeypatch.setattr(evaluate, "test", functools.partial(evaluate.test, runs=5))
    out = tmp_path / "r.json"
    assert evaluate.main(["--m", model, "--t", variant, "--o", "2", "--json", str(out)]) == 0
    r = json.loads(out.read_text())
    assert r["match"] and r["execution_time_ms"] > 0 and r["eager_time_ms"] > 0
    assert len(r["max_abs_diff"]) == {"keyformer": 2, "roco": 3}.get(variant, 1)
