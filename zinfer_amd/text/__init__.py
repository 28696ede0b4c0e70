"""The text front end: optional, only in use when a model folder brings a tokenizer.  The
engine itself takes and returns token ids."""
from .bpe import Tokenizer, TokenizerError
from .chat import (Message, ToolCall, analyze_generated_text, effective_stop_sequences,
                   render_messages, render_single_user, strip_historical_thinking)

__all__ = ["Tokenizer", "TokenizerError", "Message", "ToolCall", "render_messages",
           "render_single_user", "strip_historical_thinking", "analyze_generated_text",
           "effective_stop_sequences"]
