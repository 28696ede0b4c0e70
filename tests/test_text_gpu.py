"""Text in, text out through the command line on the GPU: a tiny random model whose
vocabulary is the synthetic tokenizer's, the chat template, stop sequences, and a batch of
requests from a file."""
import json
import os

import pytest
import torch

import text_fixture
import tiny
from gpu_util import DEV
from zinfer_amd import cli
from zinfer_amd.config import Qwen3Config
from zinfer_amd.text import Tokenizer, analyze_generated_text, render_single_user
from zinfer_amd.weights import write_model_dir

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def model_dir(tmp_path_factory):
    vocab, _, specials = text_fixture.build()
    raw = dict(tiny.CONFIGS["B"])
    raw["vocab_size"] = len(vocab) + len(specials)
    path = str(tmp_path_factory.mktemp("text_model"))
    write_model_dir(path, Qwen3Config.from_dict(raw), seed=4, dtype=torch.float32)
    text_fixture.write_tokenizer_json(path)
    return path


def _greedy(model_dir, ids, n):
    from zinfer_amd.entrypoints import LLM
    from zinfer_amd.sampling import SamplingParams
    llm = LLM(model_dir, dtype="float32", device=DEV, max_tokens=512)
    return llm.generate([ids], SamplingParams(temperature=0.0, max_new_tokens=n))[0]


def test_generate_from_text(model_dir, capsys):
    tok = Tokenizer.from_dir(model_dir)
    prompt = render_single_user("Hello world", thinking=False, system="Hi")
    want_ids = _greedy(model_dir, tok.encode(prompt), 12)
    want = tok.decode(want_ids)
    _, hit, n = analyze_generated_text(want, ["<|im_end|>"])
    for extra in ([], ["--stream"]):
        rc = cli.main(["generate", model_dir, "Hello world", "12", "no-think", "--temperature", "0",
                       "--repetition-penalty", "1", "--system", "Hi", "--dtype", "float32"] + extra)
        out = capsys.readouterr().out
        assert rc == 0
        assert out.startswith("Zinfer generate\nmode: no-think\nprompt: Hello world\nresponse: ")
        assert out[len("Zinfer generate\nmode: no-think\nprompt: Hello world\nresponse: "):] == want[:n] + "\n"
    # a stop sequence of the user's, looked for at the end of the text after every token as the
    # reference does: the answer ends before it
    pieces = [tok.decode(want_ids[:k]) for k in range(len(want_ids) + 1)]
    stop = pieces[4][len(pieces[3]):]
    if stop.strip("�"):
        expect = next(t[:analyze_generated_text(t, [stop])[2]] for t in pieces
                      if analyze_generated_text(t, [stop])[1])
        rc = cli.main(["generate", model_dir, "Hello world", "12", "--temperature", "0",
                       "--repetition-penalty", "1", "--system", "Hi", "--dtype", "float32",
                       "--stop", stop])
        out = capsys.readouterr().out
        assert rc == 0 and out.split("response: ", 1)[1] == expect + "\n"
        assert len(expect) < len(want[:n])


def test_generate_chat_and_serve_batch(model_dir, tmp_path, capsys):
    tok = Tokenizer.from_dir(model_dir)
    messages = [{"role": "user", "content": "Hi"}, {"role": "assistant", "content": "Hello"},
                {"role": "user", "content": "test"}]
    mpath = tmp_path / "messages.json"
    mpath.write_text(json.dumps(messages))
    rc = cli.main(["generate-chat", model_dir, str(mpath), "6", "think", "--temperature", "0",
                   "--repetition-penalty", "1", "--dtype", "float32"])
    out = capsys.readouterr().out
    assert rc == 0 and out.startswith("Zinfer generate-chat\nmode: think\n")
    from zinfer_amd.text import Message, render_messages
    prompt = render_messages([Message(m["role"], m["content"]) for m in messages], True)
    want = tok.decode(_greedy(model_dir, tok.encode(prompt), 6))
    _, _, n = analyze_generated_text(want, ["<|im_end|>"])
    assert out.split("response: ", 1)[1] == want[:n] + "\n"
    # a file of requests, ids and text mixed, through the scheduler
    reqs = [{"id": "a", "prompt": [5, 6, 7, 8], "max_new_tokens": 5},
            {"id": "b", "text": "Hello world", "max_new_tokens": 9, "ignore_eos": True},
            {"id": "c", "prompt": [9] * 40, "max_new_tokens": 3, "temperature": 0.8, "top_k": 5, "seed": 2}]
    rpath, opath = tmp_path / "requests.jsonl", tmp_path / "out.jsonl"
    rpath.write_text("\n".join(json.dumps(r) for r in reqs) + "\n")
    rc = cli.main(["serve-batch", model_dir, "--requests", str(rpath), "--out", str(opath),
                   "--dtype", "float32", "--max-step-tokens", "16", "--chunk", "8"])
    assert rc == 0
    got = {r["id"]: r for r in map(json.loads, opath.read_text().splitlines())}
    assert set(got) == {"a", "b", "c"}
    assert got["a"]["tokens"] == _greedy(model_dir, [5, 6, 7, 8], 5)
    assert got["b"]["tokens"] == _greedy(model_dir, tok.encode("Hello world"), 9)
    assert got["b"]["text"] == tok.decode(got["b"]["tokens"]) and len(got["c"]["tokens"]) == 3
    assert "serve-batch: 3 requests" in capsys.readouterr().err
    rpath.write_text(json.dumps({"id": 1, "prompt": [1], "text": "x"}) + "\n")
    assert cli.main(["serve-batch", model_dir, "--requests", str(rpath)]) == 1


def test_chat_turns_history_and_sessions(model_dir, tmp_path, capsys, monkeypatch):
    """`zinfer chat` over lines of standard input (`src/app/cli/chat.zig:226-312`): every turn
    is the whole history rendered anew, an earlier answer enters it as the family keeps it,
    /clear empties it, /save, /load and --save write and read sessions."""
    import io
    import sys
    from zinfer_amd.text import Message, render_messages, strip_historical_thinking
    from zinfer_amd.text.chat import load_messages
    tok = Tokenizer.from_dir(model_dir)

    def answer(history):
        text = tok.decode(_greedy(model_dir, tok.encode(render_messages(history, False)), 6))
        return text[:analyze_generated_text(text, ["<|im_end|>"])[2]]

    first = answer([Message("system", "Hi"), Message("user", "Hello")])
    history = [Message("system", "Hi"), Message("user", "Hello"),
               Message("assistant", strip_historical_thinking(first)), Message("user", "test")]
    second = answer(history)
    alone = answer([Message("system", "Hi"), Message("user", "test")])
    mid, end = tmp_path / "mid.json", tmp_path / "end.json"
    lines = ["Hello", "", f"/save {mid}", "test", "/clear", "test", f"/load {mid}", "test", "/quit",
             "never read"]
    monkeypatch.setattr(sys, "stdin", io.StringIO("\n".join(lines) + "\n"))
    rc = cli.main(["chat", model_dir, "6", "no-think", "--temperature", "0",
                   "--repetition-penalty", "1", "--system", "Hi", "--dtype", "float32",
                   "--save", str(end)])
    out = capsys.readouterr().out
    assert rc == 0
    assert out.startswith(f"Zinfer chat\nmodel_dir: {model_dir}\nmode: no-think\n"
                          "commands: /exit /quit /clear /save <path> /load <path>\n")
    said = [piece.split("\n")[0] for piece in out.split("assistant> ")[1:]]
    assert said == [first.split("\n")[0], second.split("\n")[0], alone.split("\n")[0],
                    second.split("\n")[0]]
    assert f"saved: {mid}" in out and "history cleared" in out and f"loaded: {mid}" in out
    assert [(m.role, m.content) for m in load_messages(str(mid))] == \
        [(m.role, m.content) for m in history[:3]]
    kept = load_messages(str(end))
    assert [m.role for m in kept] == ["system", "user", "assistant", "user", "assistant"]
    assert kept[-1].content == strip_historical_thinking(second)
    # a session is a start as well: the answer to the same question is the same again
    monkeypatch.setattr(sys, "stdin", io.StringIO("test\n"))
    rc = cli.main(["chat", model_dir, "6", "--temperature", "0", "--repetition-penalty", "1",
                   "--dtype", "float32", "--load", str(mid), "--stream"])
    out = capsys.readouterr().out
    assert rc == 0 and out.split("assistant> ")[1].split("\n")[0] == second.split("\n")[0]
