"""The chat format over token ids against the reference's layout
(J/model/format/LlamaChatFormat.java:41-74), with a toy tokenizer."""
import pytest

from gpullama3_java_amd.chat import ASSISTANT, SYSTEM, USER, LlamaChatFormat, Message


class ToyTokenizer:
    """One id per character (below 200), the special pieces above."""
    SPECIAL = {"<|begin_of_text|>": 200, "<|start_header_id|>": 201, "<|end_header_id|>": 202, "<|eot_id|>": 203,
               "<|end_of_text|>": 204}

    def __init__(self, special=None):
        self.special = dict(self.SPECIAL if special is None else special)

    def encode(self, text):
        return [ord(c) % 200 for c in text]

    def decode(self, ids):
        return "".join(chr(i) for i in ids if i < 200)

    def token_to_id(self, piece):
        return self.special.get(piece)


def ids(text):
    return [ord(c) % 200 for c in text]


def test_header_and_message_layout():
    f = LlamaChatFormat(ToyTokenizer())
    assert f.encode_header(Message(USER, "ignored")) == [201] + ids("user") + [202] + ids("\n")
    # the text is stripped, the turn closed (LlamaChatFormat.java:55-60)
    assert f.encode_message(Message(SYSTEM, "  be brief \n")) == [201] + ids("system") + [202] + ids("\n") + ids("be brief") + [203]


def test_dialog_prompt_and_stop_tokens():
    f = LlamaChatFormat(ToyTokenizer())
    dialog = [Message(SYSTEM, "s"), Message(USER, "u")]
    want = [200] + f.encode_message(dialog[0]) + f.encode_message(dialog[1])
    assert f.encode_dialog_prompt(False, dialog) == want
    assert f.encode_dialog_prompt(True, dialog) == want + f.encode_header(Message(ASSISTANT, ""))
    assert f.stop_tokens == frozenset((203, 204))          # end of turn, end of text (LlamaChatFormat.java:30)
    assert f.end_of_message is None                        # only Llama 3.1 has it


def test_a_vocabulary_without_the_special_pieces_is_refused():
    special = dict(ToyTokenizer.SPECIAL)
    del special["<|eot_id|>"]
    with pytest.raises(ValueError, match="eot_id"):
        LlamaChatFormat(ToyTokenizer(special))
    special = dict(ToyTokenizer.SPECIAL, **{"<|eom_id|>": 205})
    assert LlamaChatFormat(ToyTokenizer(special)).end_of_message == 205
