"""Prompt rendering and stop handling for the Qwen3 family as the reference does them
(`src/model/families/qwen3/chat_template.zig`, `src/app/cli/prompts.zig`,
`src/app/cli/runtime/streaming.zig`, `src/model/runtime/decoder_family.zig:168-200`)."""
from __future__ import annotations

import json
from dataclasses import dataclass, field
from typing import List, Optional, Sequence, Tuple


@dataclass
class ToolCall:
    name: str
    arguments_json: str


@dataclass
class Message:
    role: str                      # system | user | assistant | tool
    content: str
    tool_calls: List[ToolCall] = field(default_factory=list)


def strip_historical_thinking(content: str) -> str:
    """What follows the first ``</think>``, without leading newlines (`chat_template.zig:119-123`)."""
    at = content.find("</think>")
    return content if at < 0 else content[at + len("</think>"):].lstrip("\n")


def render_messages(messages: Sequence[Message], thinking: bool) -> str:
    """`chat_template.zig:21-44`: every message in ``<|im_start|>role\\n...<|im_end|>\\n``, tool
    results gathered in a user wrapper (`:91-106`), an assistant's earlier thinking dropped
    (`:59-62`), then the opening of the answer; without thinking an empty think block."""
    out: List[str] = []
    for i, m in enumerate(messages):
        if m.role == "tool":
            first = i == 0 or messages[i - 1].role != "tool"
            last = i + 1 == len(messages) or messages[i + 1].role != "tool"
            if first:
                out.append("<|im_start|>user")
            out.append("\n<tool_response>\n" + m.content + "\n</tool_response>")
            if last:
                out.append("<|im_end|>\n")
            continue
        content = strip_historical_thinking(m.content) if m.role == "assistant" else m.content
        out.append("<|im_start|>" + m.role + "\n" + content)
        if m.role == "assistant":
            for k, call in enumerate(m.tool_calls):
                if (k == 0 and content) or k != 0:
                    out.append("\n")
                out.append('<tool_call>\n{"name": ' + json.dumps(call.name, ensure_ascii=False)
                           + ', "arguments": ' + call.arguments_json + "}\n</tool_call>")
        out.append("<|im_end|>\n")
    out.append("<|im_start|>assistant\n")
    if not thinking:
        out.append("<think>\n\n</think>\n\n")
    return "".join(out)


def render_single_user(user_text: str, thinking: bool, system: Optional[str] = None) -> str:
    """`prompts.zig:4-21`."""
    messages = [Message("user", user_text)]
    if system is not None:
        messages.insert(0, Message("system", system))
    return render_messages(messages, thinking)


def with_system(messages: Sequence[Message], system: Optional[str]) -> List[Message]:
    """``--system`` goes first unless the messages bring their own (`prompts.zig:23-46`)."""
    messages = list(messages)
    if system is not None and (not messages or messages[0].role != "system"):
        messages.insert(0, Message("system", system))
    return messages


def load_messages(path: str) -> List[Message]:
    """A JSON list of {role, content, tool_calls?: [{name, arguments}]}, or an object that
    holds such a list under ``messages`` (a saved chat session) (`src/app/cli/messages.zig:
    13-68`)."""
    with open(path, "r", encoding="utf-8") as f:
        raw = json.load(f)
    if isinstance(raw, dict):
        raw = raw.get("messages")
    if not isinstance(raw, list):
        raise ValueError("InvalidMessages: a JSON list of messages is needed")
    out = []
    for m in raw:
        role = m.get("role")
        if role not in ("system", "user", "assistant", "tool"):
            raise ValueError(f"InvalidMessages: role {role!r}")
        calls = [ToolCall(c["name"], c["arguments"] if isinstance(c["arguments"], str)
                          else json.dumps(c["arguments"], ensure_ascii=False))
                 for c in m.get("tool_calls", [])]
        out.append(Message(role, m.get("content") or "", calls))
    return out


def effective_stop_sequences(defaults: Sequence[str], extra: Sequence[str]) -> List[str]:
    """The family's defaults, then the user's, each once, empty ones dropped
    (`decoder_family.zig:168-200`)."""
    out: List[str] = []
    for s in list(defaults) + list(extra):
        if s and s not in out:
            out.append(s)
    return out


def analyze_generated_text(text: str, stops: Sequence[str]) -> Tuple[int, bool, int]:
    """(printable_len, stop_hit, response_len) (`streaming.zig:11-39`): a stop sequence at the
    end ends the answer and is cut off; otherwise the longest tail that could still grow into
    a stop sequence is held back from printing."""
    hold = 0
    for s in stops:
        if not s:
            continue
        if text.endswith(s):
            return len(text) - len(s), True, len(text) - len(s)
        for overlap in range(min(len(text), len(s) - 1), 0, -1):
            if text[len(text) - overlap:] == s[:overlap]:
                hold = max(hold, overlap)
                break
    return len(text) - hold, False, len(text)
