"""The command line where no GPU is needed: the random-weights mode, and what it says about folders that are no model."""
import json
import os

from arle_amd.cli import main
from tiny import TINY_A, ARCH


def test_random_weights_mode_writes_a_model_folder(tmp_path, capsys):
    config = tmp_path / "config.json"
    config.write_text(json.dumps(dict(TINY_A, architectures=[ARCH])))
    out = str(tmp_path / "model")
    assert main(["random-weights", "--config", str(config), "--out", out, "--seed-weights", "3"]) == 0
    assert capsys.readouterr().out.strip() == out
    assert sorted(os.listdir(out)) == ["config.json", "model.safetensors"]
    assert json.load(open(os.path.join(out, "config.json")))["hidden_size"] == TINY_A["hidden_size"]


def test_a_folder_that_is_no_model_ends_in_one_line_and_exit_code_1(tmp_path, capsys):
    assert main(["--model-path", str(tmp_path / "nothing"), "run", "--prompt-ids", "1,2"]) == 1
    err = capsys.readouterr().err.strip().splitlines()
    assert len(err) == 1 and err[0].startswith("error: ") and "config.json" in err[0]
    (tmp_path / "config.json").write_text(json.dumps(dict(TINY_A, architectures=[ARCH], num_hidden_layers=10 ** 12)))
    assert main(["--model-path", str(tmp_path), "run", "--prompt-ids", "1,2"]) == 1
    assert "num_hidden_layers" in capsys.readouterr().err
    assert main(["run", "--prompt-ids", "1,2"]) == 2      # no model named at all: a usage error
