"""What a prompt is made of beside text: control tokens by name, and the messages of a chat.

A prompt is a string, a list of token ids, or a list of blocks: text, token ids and
``ControlToken``s (python/libllm/__init__.py:46-111 of the reference).  How the messages of a
conversation become such a list is the architecture's business: its configuration class may have
``build_prompt(messages)``; the entry points fall back to ``plain_prompt`` where the tokenizer
beside the model does not know the control tokens (or there is none and bytes serve as tokens).
"""
from typing import Dict, List, Sequence, Union

from .errors import RequestError


class ControlToken:
    """A control token in a prompt, by name, for example <|eot_id|>."""

    def __init__(self, token_name: str) -> None:
        self._name = token_name

    def __repr__(self) -> str:
        return "ControlToken(%r)" % self._name

    def __eq__(self, other) -> bool:
        return isinstance(other, ControlToken) and other._name == self._name

    def __hash__(self) -> int:
        return hash(("control", self._name))


Block = Union[str, int, ControlToken]


def check_messages(messages: Sequence[Dict[str, str]]) -> None:
    """Messages are ``{"role", "content"}``; the last one is the user's, or the assistant's to be
    continued (src/libllm/llama.cc:406-442, src/libllm/llm.cc:98-123)."""
    if not messages:
        raise RequestError("history is empty")
    for m in messages:
        if not isinstance(m, dict) or "role" not in m or "content" not in m:
            raise RequestError("a message needs \"role\" and \"content\"")
    if messages[-1]["role"] not in ("user", "assistant"):
        raise RequestError("invalid messages: role of last message should be either user or assistant")


def plain_prompt(messages: Sequence[Dict[str, str]]) -> str:
    """The messages as lines of text, for a model without control tokens."""
    check_messages(messages)
    text = "".join("%s: %s\n" % (m["role"], m["content"]) for m in messages[:-1])
    last = messages[-1]
    if last["role"] == "user":
        return text + "%s: %s\nassistant: " % (last["role"], last["content"])
    return text + "%s: %s" % (last["role"], last["content"])


def llama3_prompt(messages: Sequence[Dict[str, str]]) -> List[Block]:
    """The Llama 3 chat format, block by block as the reference's model class appends them
    (src/libllm/llama.cc:406-442): every earlier message between its header and <|eot_id|>, the
    last one, if the user's, followed by the assistant's open header; if the assistant's, left
    open so that the reply continues it."""
    check_messages(messages)

    def header(role):
        return [ControlToken("<|start_header_id|>"), role, ControlToken("<|end_header_id|>")]
    blocks: List[Block] = [ControlToken("<|begin_of_text|>")]
    for m in messages[:-1]:
        blocks += header(m["role"]) + ["\n\n" + m["content"], ControlToken("<|eot_id|>")]
    last = messages[-1]
    blocks += header(last["role"]) + ["\n\n" + last["content"]]
    if last["role"] == "user":
        blocks += [ControlToken("<|eot_id|>")] + header("assistant") + ["\n\n"]
    return blocks
