"""Named shapes parse as configurations of the architecture, and the command line writes them."""
import json

from nano_vllm_amd.cli import main
from nano_vllm_amd.config import architecture_of
from nano_vllm_amd.models.shapes import SHAPES, shape


def test_named_shapes_are_valid_configurations():
    for name in SHAPES:
        cj = shape(name)
        cfg = architecture_of(cj).parse_config(cj)
        assert cfg.num_attention_heads % cfg.num_key_value_heads == 0
        assert cfg.to_dict()["hidden_size"] == cj["hidden_size"]
    big = architecture_of(shape("qwen3-8b")).parse_config(shape("qwen3-8b"))
    assert (big.num_hidden_layers, big.hidden_size, big.intermediate_size, big.vocab_size) == (36, 4096, 12288, 151936)


def test_random_model_command_writes_a_shape(tmp_path, capsys):
    assert main(["random-model", "--shape", "qwen3-32b", "--config-only", "--out", str(tmp_path / "c")]) == 0
    cj = json.loads((tmp_path / "c" / "config.json").read_text())
    assert cj["num_hidden_layers"] == 64 and not (tmp_path / "c" / "model.safetensors").exists()
    assert main(["random-model", "--shape", "tiny-b", "--seed", "2", "--out", str(tmp_path / "m")]) == 0
    assert (tmp_path / "m" / "model.safetensors").exists()
    assert main(["random-model", "--out", str(tmp_path / "x")]) == 2


def test_throughput_command_refuses_an_empty_range_of_lengths(capsys):
    assert main(["throughput", "--model", "nowhere", "--max-output-len", "64"]) == 2       # the minimum's default is 100
    assert "--min-output-len 100 and --max-output-len 64" in capsys.readouterr().err
    assert main(["throughput", "--model", "nowhere", "--min-input-len", "0"]) == 2
