"""The command line: the reference's positional forms, flags, presets and error names
(src/app/cli/args.zig), on the CPU; generation through it runs on the GPU."""
import json
import subprocess
import sys
import os

import pytest
import torch

import plain
import tiny
from zinfer_amd import cli

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_token_ids_csv():
    """src/app/cli/token_ids.zig:3-18"""
    assert cli.parse_token_ids("1, 2,3,,4 ") == [1, 2, 3, 4]
    with pytest.raises(cli.CliError):
        cli.parse_token_ids("1,x")


def test_generate_positional_forms_and_presets():
    d, ids, opt = cli.parse_generate(["1,2,3"], 64)
    assert (d, ids, opt.max_new_tokens, opt.think) == (cli.DEFAULT_MODEL_DIR, [1, 2, 3], 64, False)
    assert (opt.sampling.temperature, opt.sampling.top_k, opt.sampling.top_p,
            opt.sampling.repetition_penalty) == (0.7, 20, 0.8, 1.1)
    d, ids, opt = cli.parse_generate(["some/dir", "1,2", "9", "think", "--seed", "7"], 64)
    assert (d, ids, opt.max_new_tokens, opt.think, opt.seed) == ("some/dir", [1, 2], 9, True, 7)
    assert (opt.sampling.temperature, opt.sampling.top_p) == (0.6, 0.95)
    d, ids, opt = cli.parse_generate(["1,2", "5", "--temperature", "0", "--top-k", "3",
                                      "--min-p", "0.1", "--ignore-eos"], 64)
    assert d == cli.DEFAULT_MODEL_DIR and opt.max_new_tokens == 5
    assert opt.sampling.temperature == 0.0 and opt.sampling.top_k == 3 and opt.sampling.ignore_eos
    assert opt.sampling.max_new_tokens == 5


@pytest.mark.parametrize("args,word", [
    (["1,2", "--temperature"], "MissingFlagValue"), (["1,2", "--frobnicate", "1"], "UnknownFlag"),
    (["1,2", "5", "maybe"], "InvalidThinkingMode"), (["1,2", "--backend", "q8"], "InvalidBackendScheme"),
    (["1,2", "--kv-cache", "q8"], "InvalidKvCacheScheme"), ([], "InvalidCommand")])
def test_errors_carry_the_reference_names(args, word):
    with pytest.raises(cli.CliError, match=word):
        cli.parse_generate(args, 64)


def test_inspect_and_random_model(tmp_path, capsys):
    cfg_path = tmp_path / "c.json"
    cfg_path.write_text(json.dumps(tiny.TINY_A))
    out = tmp_path / "model"
    assert cli.main(["random-model", str(cfg_path), str(out), "--seed", "3", "--dtype", "float32"]) == 0
    assert cli.main(["inspect-config", str(out)]) == 0
    text = capsys.readouterr().out
    assert "model_type: qwen3" in text and "head_dim: 16" in text and "architecture: Qwen3ForCausalLM" in text
    assert cli.main(["inspect-weights", str(out)]) == 0
    assert "tensor_count: 24" in capsys.readouterr().out
    assert cli.main(["inspect-tensor", str(out), "model.norm.weight", "3"]) == 0
    assert "shape=[64]" in capsys.readouterr().out
    assert cli.main(["inspect-tensor", str(out), "nope"]) == 1
    assert cli.main(["frobnicate"]) == 2 and cli.main(["quantize", "q8"]) == 2


@pytest.mark.gpu
def test_generate_token_ids_through_the_command_line(tmp_path):
    path = tiny.model_dir_of("B", str(tmp_path), torch.float32)
    prompt = tiny.random_tokens(11, 1000, 8)
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "zinfer"), "generate-token-ids",
                        path, ",".join(map(str, prompt)), "6", "--dtype", "float32",
                        "--page-size", "8"], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr
    line = [l for l in r.stdout.splitlines() if l.startswith("tokens: ")][0]
    got = json.loads(line[len("tokens: "):])
    want = prompt + plain.greedy_generate(tiny.CONFIGS["B"], tiny.weights_of("B"), prompt, 6)
    assert got == want


@pytest.mark.gpu
def test_random_weights_without_a_model_folder(tmp_path):
    """``--config f --random-weights S`` and ``LLM.from_config`` draw what ``write_model_dir``
    stores for the same seed, so the plain implementation over those tensors is the oracle."""
    from zinfer_amd import LLM, SamplingParams
    prompt = tiny.random_tokens(9, 512, 3)
    want = plain.greedy_generate(tiny.CONFIGS["A"], tiny.weights_of("A"), prompt, 5)
    llm = LLM.from_config(tiny.CONFIGS["A"], seed=tiny.SEEDS["A"], dtype="float32",
                          max_tokens=128, max_seqs=2)
    got = llm.generate([prompt], SamplingParams(temperature=0.0, max_new_tokens=5,
                                                ignore_eos=True))[0]
    assert got == want
    cfg = tmp_path / "config.json"
    cfg.write_text(json.dumps(tiny.CONFIGS["A"]))
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "zinfer"), "generate-token-ids",
                        ",".join(map(str, prompt)), "5", "--dtype", "float32", "--config",
                        str(cfg), "--random-weights", str(tiny.SEEDS["A"])],
                       capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr
    line = [l for l in r.stdout.splitlines() if l.startswith("tokens: ")][0]
    assert json.loads(line[len("tokens: "):]) == prompt + want


def test_config_and_random_weights_go_together():
    from zinfer_amd.cli import CliError, Options, _llm, parse_flags
    opt = Options(4)
    parse_flags(["--config", "x.json"], opt)
    with pytest.raises(CliError, match="go together"):
        _llm("nowhere", opt)
