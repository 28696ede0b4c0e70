"""The text front end against what the reference's own tests and sources fix: the byte table,
the hand-written pre-token rules, merge order, special tokens, the chat template and the stop
analysis (src/tokenizer/bpe.zig, src/tokenizer/bpe/*.zig,
src/model/families/qwen3/chat_template.zig, src/app/cli/runtime/streaming.zig)."""
import pytest

import text_fixture
from zinfer_amd import cli
from zinfer_amd.text import (Message, Tokenizer, TokenizerError, ToolCall, analyze_generated_text,
                             effective_stop_sequences, render_messages, render_single_user,
                             strip_historical_thinking)
from zinfer_amd.text.bpe import byte_table, pre_tokens, utf8_lossy


def test_byte_table():
    """bpe/byte_mapping.zig:13-44: printable bytes stand for themselves, the other 68 take
    256.. in byte order: 0 -> U+0100, newline (the 11th of them) -> U+010A, space -> U+0120."""
    enc, dec = byte_table()
    assert enc[ord("!")] == "!" and enc[ord("~")] == "~" and enc[0xA1] == "¡" and enc[0xFF] == "ÿ"
    assert enc[0] == "Ā" and enc[10] == "Ċ" and enc[32] == "Ġ" and enc[0xAD] == "Ń"
    assert len(set(enc)) == 256 and all(dec[c] == b for b, c in enumerate(enc))


def _cut(text, specials=()):
    return [p for p, _ in pre_tokens(text, list(specials))]


def test_pre_token_rules():
    """bpe/pretokenize.zig:16-158, rule by rule."""
    assert _cut("Hello world") == ["Hello", " world"]                      # space goes with the word
    assert _cut("a   b") == ["a", "  ", " b"]                              # all spaces but the last alone
    assert _cut("x \t") == ["x", " \t"]                                    # trailing blanks: one run
    assert _cut("don't I'LL") == ["don", "'t", " I", "'LL"]                 # contractions, any case
    assert _cut("it's'x") == ["it", "'s", "'", "x"]                        # a lone quote is punctuation
    assert _cut("abc12345 678") == ["abc", "12345", " ", "678"]            # digit runs of any length
    assert _cut("wait...\n\nnext") == ["wait", "...\n\n", "next"]          # punctuation takes newlines
    assert _cut("a ?!\nb") == ["a", " ?!\n", "b"]                          # one space + punctuation
    assert _cut("a\r\n\nb") == ["a", "\r\n\n", "b"]                        # newline runs
    assert _cut("你好，世界") == ["你好", "，", "世界"]   # CJK letters, wide comma
    assert _cut("été мир") == ["été", " мир"]
    # a special token ends every run and is cut out whole, the longest one first
    sp = ["<|im_end|>", "<|im", "<think>"]
    assert pre_tokens("ab<|im_end|>\n<think>x", sp) == [
        ("ab", False), ("<|im_end|>", True), ("\n", False), ("<think>", True), ("x", False)]
    assert "".join(_cut(" mixed 12 !? \n\t end  ")) == " mixed 12 !? \n\t end  "


@pytest.fixture(params=["tokenizer.json", "reference files"])
def tok(request, tmp_path):
    if request.param == "tokenizer.json":
        text_fixture.write_tokenizer_json(str(tmp_path))
    else:
        text_fixture.write_reference_files(str(tmp_path))
    return Tokenizer.from_dir(str(tmp_path))


def test_encode_and_decode_known_shapes(tok):
    """The shapes of the reference's vectors (bpe.zig:180-213) on the synthetic vocabulary:
    'Hello' and ' hello' are one token each, special tokens come out whole, a newline is the
    byte symbol U+010A."""
    v, s = tok.vocab, tok.specials
    assert tok.encode("Hello") == [v["Hello"]]
    assert tok.encode(" hello") == [v["Ġhello"]]
    chat = "<|im_start|>user\nHello<|im_end|>\n"
    ids = tok.encode(chat)
    assert ids == [s["<|im_start|>"], v["user"], v["Ċ"], v["Hello"], s["<|im_end|>"], v["Ċ"]]
    assert tok.encode("<think>test</think>") == [s["<think>"], v["test"], s["</think>"]]
    assert tok.decode(ids) == chat
    # the thinking-off prompt ends in two double newlines (chat_template.zig:143-158)
    ids = tok.encode(render_single_user("Hello", thinking=False))
    assert ids[-4:] == [s["<think>"], v["ĊĊ"], s["</think>"], v["ĊĊ"]]
    # anything the merges do not cover falls back to byte symbols and still round-trips
    for text in ["Hello, wor1d! 12345\n\té你\U0001f600 end", " a  b   c", "'s'T x"]:
        assert tok.decode(tok.encode(text)) == text


def test_merges_apply_lowest_rank_first():
    """bpe/merge.zig:17-34: the lowest rank anywhere wins, the leftmost among equal ranks."""
    enc, _ = byte_table()
    vocab = {c: i for i, c in enumerate(enc)}
    for t in ("ab", "bc", "abc", "aa"):
        vocab[t] = len(vocab)
    t1 = Tokenizer(vocab, ["b c", "a b", "a bc"], {})
    assert t1.encode("abc") == [vocab["abc"]]                 # b+c first, then a+bc
    t2 = Tokenizer(vocab, ["a b", "b c", "a bc"], {})
    assert t2.encode("abc") == [vocab["ab"], vocab["c"]]      # a+b first; (ab, c) has no rank
    t3 = Tokenizer(vocab, ["# a comment", "a a"], {})
    assert t3.encode("aaa") == [vocab["aa"], vocab["a"]]      # leftmost pair of equal rank
    with pytest.raises(TokenizerError, match="TokenNotFound"):
        Tokenizer({c: i for i, c in enumerate(enc)}, ["a b"], {}).encode("ab")


def test_decode_errors_and_lossy_utf8(tok):
    with pytest.raises(TokenizerError, match="UnknownTokenId"):
        tok.decode([10 ** 6])
    # the first two bytes of a three-byte character: neither starts a valid sequence
    assert tok.decode([0xE4, 0xBD]) == "��"
    assert utf8_lossy(b"ok\xffok\xe4\xbd\xa0") == "ok�ok你"
    assert tok.decode([0xE4, 0xBD, 0xA0]) == "你"


def test_chat_template_vectors():
    """chat_template.zig:125-222."""
    assert render_single_user("Hello", True) == "<|im_start|>user\nHello<|im_end|>\n<|im_start|>assistant\n"
    assert render_single_user("Hello", False) == \
        "<|im_start|>user\nHello<|im_end|>\n<|im_start|>assistant\n<think>\n\n</think>\n\n"
    messages = [Message("system", "You are terse."), Message("user", "Hi"),
                Message("assistant", "<think>\ninternal\n</think>\nHello there"), Message("user", "Next")]
    assert render_messages(messages, False) == (
        "<|im_start|>system\nYou are terse.<|im_end|>\n<|im_start|>user\nHi<|im_end|>\n"
        "<|im_start|>assistant\nHello there<|im_end|>\n<|im_start|>user\nNext<|im_end|>\n"
        "<|im_start|>assistant\n<think>\n\n</think>\n\n")
    call = Message("assistant", "", [ToolCall("lookup_weather", '{"city":"Shanghai"}')])
    assert render_messages([call], True) == (
        "<|im_start|>assistant\n<tool_call>\n{\"name\": \"lookup_weather\", \"arguments\": "
        "{\"city\":\"Shanghai\"}}\n</tool_call><|im_end|>\n<|im_start|>assistant\n")
    tools = [Message("tool", '{"ok":true}'), Message("tool", '{"temp":22}')]
    assert render_messages(tools, True) == (
        "<|im_start|>user\n<tool_response>\n{\"ok\":true}\n</tool_response>\n<tool_response>\n"
        "{\"temp\":22}\n</tool_response><|im_end|>\n<|im_start|>assistant\n")
    assert strip_historical_thinking("no tags") == "no tags"
    assert render_single_user("Q", True, system="S").startswith("<|im_start|>system\nS<|im_end|>\n")


def test_stop_analysis_vectors():
    """streaming.zig:67-86 and decoder_family.zig:357-364."""
    assert analyze_generated_text("Hello today?", ["today?"]) == (6, True, 6)
    assert analyze_generated_text("Hello to", ["today?"]) == (6, False, 8)
    assert analyze_generated_text("Hello", ["", "xyz"]) == (5, False, 5)
    assert effective_stop_sequences(["<|im_end|>"], ["</tool_response>", "<|im_end|>"]) == \
        ["<|im_end|>", "</tool_response>"]


def test_tokenize_and_decode_ids_commands(tmp_path, capsys):
    """src/app/cli/tools/text.zig:5-75: the printed form."""
    import json
    import tiny
    text_fixture.write_tokenizer_json(str(tmp_path))
    # the tokenizer is the one of the architecture that config.json names (text.zig:10-20)
    (tmp_path / "config.json").write_text(json.dumps(tiny.TINY_A))
    vocab, _, specials = text_fixture.build()
    assert cli.main(["tokenize", str(tmp_path), "Hello<|im_end|>"]) == 0
    out = capsys.readouterr().out
    assert out == f"Zinfer tokenize\ntext: Hello<|im_end|>\nids: [{vocab['Hello']}, {specials['<|im_end|>']}]\n"
    assert cli.main(["decode-ids", str(tmp_path), f"{vocab['Hi']},{vocab[chr(0x120) + 'world']}"]) == 0
    assert capsys.readouterr().out.endswith("text: Hi world\n")
    assert cli.main(["tokenize", str(tmp_path / "nothing"), "x"]) == 1
    assert "no config.json" in capsys.readouterr().err
    (tmp_path / "bare").mkdir()
    (tmp_path / "bare" / "config.json").write_text(json.dumps(tiny.TINY_A))
    assert cli.main(["tokenize", str(tmp_path / "bare"), "x"]) == 1
    assert "TokenizerNotFound" in capsys.readouterr().err
