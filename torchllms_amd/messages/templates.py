"""Chat templates as data, and the tokenisation of a conversation with one.

A template lists, per role, the text that opens and closes a message, a text that starts the
whole conversation, the text that invites the assistant's next turn, and the token ids that end
a turn.  The Llama 3 values restate
reference: torchllms/messages/configs/llama3_instruct.yaml:9-32; the region-by-region encoding
follows reference: torchllms/messages/tokenization.py:368-422 (envelopes may hold special tokens,
message content is encoded so that it cannot).
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, List, Optional, Sequence, Tuple


@dataclass(frozen=True)
class ChatTemplate:
    bos: str
    roles: Dict[str, Tuple[str, str]]  # role -> (text before the content, text after it)
    generation_prompt: str
    stop_token_ids: Tuple[int, ...]
    strip_whitespace: bool = True


def _llama3_header(role: str) -> str:
    return "<|start_header_id|>" + role + "<|end_header_id|>\n\n"


LLAMA3_INSTRUCT = ChatTemplate(
    bos="<|begin_of_text|>",
    roles={
        "system": (_llama3_header("system"), "<|eot_id|>"),
        "user": (_llama3_header("user"), "<|eot_id|>"),
        "assistant": (_llama3_header("assistant"), "<|eot_id|>"),
        "tool": (_llama3_header("ipython"), "<|eot_id|>"),
    },
    generation_prompt=_llama3_header("assistant"),
    stop_token_ids=(128009,),
)

TEMPLATES: Dict[str, ChatTemplate] = {
    "llama3_instruct": LLAMA3_INSTRUCT,
    "llama3_instruct.yaml": LLAMA3_INSTRUCT,
}


def get_template(name: Optional[str]) -> Optional[ChatTemplate]:
    if name is None:
        return None
    try:
        return TEMPLATES[name]
    except KeyError:
        raise KeyError(f"no chat template named {name!r}; known: {sorted(TEMPLATES)}") from None


def tokenize_conversation(conversation: Sequence[Dict[str, str]], tokenizer, template: ChatTemplate,
                          add_generation_prompt: bool = True) -> List[int]:
    """Token ids of a conversation (a list of ``{"role", "content"}``).  ``tokenizer`` needs
    ``encode(text)`` (special tokens in the text become their ids) and may have
    ``encode_plain(text)`` (text is never read as special tokens), used for message content."""
    plain = getattr(tokenizer, "encode_plain", tokenizer.encode)
    ids: List[int] = []
    if template.bos:
        ids += tokenizer.encode(template.bos)
    for msg in conversation:
        role = msg["role"]
        if role not in template.roles:
            raise KeyError(f"role {role!r} is not in the template; known: {sorted(template.roles)}")
        before, after = template.roles[role]
        content = msg["content"].strip() if template.strip_whitespace else msg["content"]
        ids += tokenizer.encode(before)
        ids += plain(content)
        ids += tokenizer.encode(after)
    if add_generation_prompt:
        ids += tokenizer.encode(template.generation_prompt)
    return ids


class FileTokenizer:
    """A ``tokenizer.json`` loaded with the ``tokenizers`` library."""

    def __init__(self, path):
        from tokenizers import Tokenizer

        self._tok = Tokenizer.from_file(str(path))

    def encode(self, text: str) -> List[int]:
        return self._tok.encode(text, add_special_tokens=False).ids

    def encode_plain(self, text: str) -> List[int]:
        had = getattr(self._tok, "encode_special_tokens", None)
        if had is None:
            return self.encode(text)
        self._tok.encode_special_tokens = True
        try:
            return self._tok.encode(text, add_special_tokens=False).ids
        finally:
            self._tok.encode_special_tokens = had

    def decode(self, ids: Sequence[int]) -> str:
        return self._tok.decode(list(ids), skip_special_tokens=True)
