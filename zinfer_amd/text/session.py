"""A chat session on disk: the messages so far and the options they were made with
(`src/app/cli/chat.zig:102-208`).  ``load_messages`` reads it back (it takes the list under
``messages``)."""
from __future__ import annotations

import json
import time
from typing import Dict, Sequence

from .chat import Message


def session_record(messages: Sequence[Message], model_dir: str, options: Dict) -> Dict:
    """The JSON object of a saved session: version, kind, time, the model folder, the options
    as given, and the messages with their tool calls (arguments stay JSON text)."""
    out = []
    for m in messages:
        item = {"role": m.role, "content": m.content}
        if m.tool_calls:
            item["tool_calls"] = [{"name": c.name, "arguments": c.arguments_json}
                                  for c in m.tool_calls]
        out.append(item)
    return {"version": 1, "kind": "zinfer_chat_session", "saved_unix": int(time.time()),
            "model_dir": model_dir, "options": options, "messages": out}


def save_session(path: str, messages: Sequence[Message], model_dir: str, options: Dict) -> None:
    with open(path, "w", encoding="utf-8") as f:
        json.dump(session_record(messages, model_dir, options), f, ensure_ascii=False, indent=2)
        f.write("\n")
