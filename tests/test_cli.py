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


def test_probe_positional_forms():
    """src/app/cli.zig:47-135: the model folder first when it is there, numbers left out take
    the defaults."""
    D = cli.DEFAULT_MODEL_DIR
    assert cli._probe_args([], 2, (0, 8))[:3] == (D, None, [0, 8])
    assert cli._probe_args(["7"], 2, (0, 8))[:3] == (D, None, [7, 8])
    assert cli._probe_args(["some/dir", "7", "3"], 2, (0, 8))[:3] == ("some/dir", None, [7, 3])
    assert cli._probe_args(["some/dir"], 3, (0, 0, 8))[:3] == ("some/dir", None, [0, 0, 8])
    assert cli._probe_args(["2", "5"], 3, (0, 0, 8))[:3] == (D, None, [2, 5, 8])
    assert cli._probe_args(["w.weight"], 2, (0, 8), name_first=True)[:3] == (D, "w.weight", [0, 8])
    assert cli._probe_args(["d", "w.weight", "4", "2", "--dtype", "float32"], 2, (0, 8),
                           name_first=True)[:3] == ("d", "w.weight", [4, 2])
    for bad, kw in ((["1", "2", "3"], {}), (["a", "b", "1"], {}), ([], {"name_first": True}),
                    (["a", "b", "c"], {"name_first": True})):
        with pytest.raises(cli.CliError, match="InvalidCommand"):
            cli._probe_args(bad, 2, (0, 8), **kw)


def test_chat_positional_forms_and_flags():
    """src/app/cli/args.zig:189-226,525-553"""
    d, opt = cli.parse_chat([])
    assert (d, opt.max_new_tokens, opt.think, opt.load_path, opt.save_path) == \
        (cli.DEFAULT_MODEL_DIR, 128, False, None, None)
    d, opt = cli.parse_chat(["40", "think"])
    assert (d, opt.max_new_tokens, opt.think, opt.sampling.temperature) == \
        (cli.DEFAULT_MODEL_DIR, 40, True, 0.6)
    d, opt = cli.parse_chat(["some/dir", "9", "no-think", "--load", "a.json", "--save", "b.json",
                             "--system", "Be brief."])
    assert (d, opt.max_new_tokens, opt.load_path, opt.save_path, opt.system) == \
        ("some/dir", 9, "a.json", "b.json", "Be brief.")
    assert opt.sampling.max_new_tokens == 9
    with pytest.raises(cli.CliError, match="InvalidThinkingMode"):
        cli.parse_chat(["some/dir", "9", "perhaps"])
    with pytest.raises(cli.CliError, match="UnknownFlag"):      # chat only
        cli.parse_generate(["1,2", "--load", "a.json"], 64)


def test_a_session_is_saved_and_read_back(tmp_path):
    """src/app/cli/chat.zig:315-368: what the reference's own test saves and finds again."""
    from zinfer_amd.text import Message, ToolCall
    from zinfer_amd.text.chat import load_messages
    from zinfer_amd.text.session import save_session
    history = [Message("system", "You are terse."), Message("user", "Use the weather tool."),
               Message("assistant", "", [ToolCall("lookup_weather", '{"city":"Shanghai"}')]),
               Message("tool", '{"temp":22}')]
    _, opt = cli.parse_chat(["64", "--seed", "7", "--stream", "--stop", "</tool_response>",
                             "--system", "You are terse."])
    path = tmp_path / "session.json"
    save_session(str(path), history, "models/Qwen3-0.6B", cli._session_options(opt))
    saved = json.loads(path.read_text())
    assert saved["kind"] == "zinfer_chat_session" and saved["version"] == 1
    assert saved["model_dir"] == "models/Qwen3-0.6B"
    assert saved["options"]["seed"] == 7 and saved["options"]["stream_output"] is True
    assert saved["options"]["stop_sequences"] == ["</tool_response>"]
    assert saved["options"]["sampling"]["top_k"] == 20
    assert "tool_calls" in saved["messages"][2]
    loaded = load_messages(str(path))
    assert [m.role for m in loaded] == ["system", "user", "assistant", "tool"]
    assert loaded == history
    assert loaded[2].tool_calls[0].arguments_json == '{"city":"Shanghai"}'


def _printed_numbers(out: str, key: str):
    line = [l for l in out.splitlines() if l.startswith(key)][0]
    return json.loads(line[len(key):])


@pytest.mark.gpu
def test_probe_commands_against_the_plain_parts(tmp_path, capsys):
    """probe-linear, probe-block and probe-model (src/app/cli/inspect.zig:109-244): a matrix's
    column, one block over a hidden vector that is 1 at one place, one token's largest logits,
    each against the plain implementation of that part."""
    path = tiny.model_dir_of("B", str(tmp_path), torch.float32)
    cfg, w = tiny.CONFIGS["B"], tiny.weights_of("B")
    name = "model.layers.1.mlp.down_proj.weight"
    for dtype in ("float32", "bfloat16"):
        assert cli.main(["probe-linear", path, name, "3", "5", "--dtype", dtype]) == 0
        out = capsys.readouterr().out
        assert out.startswith(f"Zinfer linear probe\ntensor: {name}\n")
        assert f"shape: {list(w[name].shape)}" in out and "input_index: 3" in out
        want = w[name][:5, 3].float()           # (stored in 32-bit: it stays so in either build)
        assert _printed_numbers(out, "first_outputs: ") == pytest.approx(want.tolist(), abs=1e-6)
    assert cli.main(["probe-linear", path, name, "999"]) == 1
    assert cli.main(["probe-linear", path, "model.norm.weight"]) == 1
    assert cli.main(["probe-linear", path, "nope"]) == 1
    err = capsys.readouterr().err
    assert "InputIndexOutOfBounds" in err and "InvalidTensorRank" in err and "TensorNotFound" in err

    hidden = torch.zeros(cfg["hidden_size"], dtype=torch.float64)
    hidden[2] = 1.0
    want = plain.block_token(cfg, w, 1, hidden, 0, [], [])
    assert cli.main(["probe-block", path, "1", "2", "6", "--dtype", "float32"]) == 0
    out = capsys.readouterr().out
    assert out.startswith("Zinfer block probe\nlayer_index: 1\ninput_index: 2\ncache_len: 1\n")
    assert _printed_numbers(out, "first_outputs: ") == pytest.approx(want[:6].tolist(), abs=2e-5)
    assert cli.main(["probe-block", path, "1", str(cfg["hidden_size"])]) == 1
    assert cli.main(["probe-block", path, str(cfg["num_hidden_layers"])]) == 1
    capsys.readouterr()

    logits = plain.model_forward(cfg, w, [5])[0]
    top = logits.topk(4)
    assert cli.main(["probe-model", path, "5", "4", "--dtype", "float32"]) == 0
    out = capsys.readouterr().out
    assert out.startswith("Zinfer model probe\ntoken_id: 5\n")
    lines = [l for l in out.splitlines() if l.startswith("top_logit ")]
    assert [int(l.split("token=")[1].split()[0]) for l in lines] == top.indices.tolist()
    assert [float(l.split("value=")[1]) for l in lines] == pytest.approx(top.values.tolist(), abs=2e-5)
    assert cli.main(["probe-model", path, str(cfg["vocab_size"])]) == 1


@pytest.mark.gpu
def test_a_probed_block_leaves_the_cache_as_it_was(tmp_path):
    """Engine.probe_block over several positions, beside a live request: its pages come from
    the pool and go back, and the live request's logits are what they are without it."""
    from zinfer_amd.engine import StepEntry
    from zinfer_amd.entrypoints import LLM
    path = tiny.model_dir_of("A", str(tmp_path), torch.float32)
    cfg, w = tiny.CONFIGS["A"], tiny.weights_of("A")
    llm = LLM(path, dtype="float32", page_size=8, max_tokens=64)
    eng = llm.engine
    toks = tiny.random_tokens(12, cfg["vocab_size"], 3)
    eng.step([StepEntry("r", toks[:7], [])])
    free = eng.cache.num_free_pages()
    T = 11
    hidden = torch.randn((T, cfg["hidden_size"]), generator=torch.Generator().manual_seed(5))
    out, held = eng.probe_block(0, hidden.cuda())
    assert held == T and eng.cache.num_free_pages() == free
    eng.cache.check()
    ks, vs = [], []
    want = torch.stack([plain.block_token(cfg, w, 0, hidden[p].double(), p, ks, vs)
                        for p in range(T)])
    assert (out.cpu().double() - want).abs().max() <= 2e-5 * want.abs().max()
    got = eng.step([StepEntry("r", toks[7:], [4])], end=["r"])[0].cpu().double()
    ref = plain.model_forward(cfg, w, toks)[-1]
    assert (got - ref).abs().max() <= 2e-5 * ref.abs().max()
