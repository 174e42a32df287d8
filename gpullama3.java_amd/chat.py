"""The Llama 3 chat format over token ids. The token protocol is fixed by the model family, so the
functions follow the reference's one for one: ``encode_header`` J/model/format/LlamaChatFormat.java:44-51,
``encode_message`` :53-59, ``encode_dialog_prompt`` :61-72, the special tokens :21-42, the roles
J/model/format/ChatFormat.java: a message is its header (start-of-header, the role's
name, end-of-header, a line feed), its stripped text and end-of-turn; a dialogue starts with
begin-of-text; generation stops at end-of-text or end-of-turn.

The tokenizer is whatever the caller has: an object with ``encode(text) -> ids`` (no special
tokens added) and ``token_to_id(piece) -> id or None``. The library itself starts at token ids.
"""
from __future__ import annotations

from dataclasses import dataclass

SYSTEM, USER, ASSISTANT = "system", "user", "assistant"


@dataclass(frozen=True)
class Message:
    role: str
    content: str


class LlamaChatFormat:
    def __init__(self, tokenizer):
        self.tokenizer = tokenizer

        def special(piece, required=True):
            tid = tokenizer.token_to_id(piece)
            if tid is None and required:
                raise ValueError(f"the tokenizer has no {piece} token: not a Llama 3 vocabulary")
            return tid

        self.begin_of_text = special("<|begin_of_text|>")
        self.start_header = special("<|start_header_id|>")
        self.end_header = special("<|end_header_id|>")
        self.end_of_turn = special("<|eot_id|>")
        self.end_of_text = special("<|end_of_text|>")
        self.end_of_message = special("<|eom_id|>", required=False)      # only in 3.1
        self.stop_tokens = frozenset((self.end_of_text, self.end_of_turn))

    def _ids(self, text):
        return list(self.tokenizer.encode(text))

    def encode_header(self, message):
        return [self.start_header] + self._ids(message.role) + [self.end_header] + self._ids("\n")

    def encode_message(self, message):
        return self.encode_header(message) + self._ids(message.content.strip()) + [self.end_of_turn]

    def encode_dialog_prompt(self, append_assistant_turn, dialog):
        tokens = [self.begin_of_text]
        for message in dialog:
            tokens += self.encode_message(message)
        if append_assistant_turn:
            tokens += self.encode_header(Message(ASSISTANT, ""))
        return tokens


class HFTokenizer:
    """A ``tokenizers.Tokenizer`` (tokenizer.json) behind the two calls the chat format needs."""

    def __init__(self, path):
        from tokenizers import Tokenizer
        self._tok = Tokenizer.from_file(path)

    def encode(self, text):
        return self._tok.encode(text, add_special_tokens=False).ids

    def decode(self, ids):
        return self._tok.decode(list(ids), skip_special_tokens=False)

    def token_to_id(self, piece):
        return self._tok.token_to_id(piece)
