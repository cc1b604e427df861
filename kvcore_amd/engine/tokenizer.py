"""Text in and out, when the model folder has a tokenizer.

Reference: kvcore/utils/tokenizer.py:15-114 (chat template with the generation prompt
appended, decode, stop ids from the tokenizer).  A folder of random weights has no
tokenizer; requests then carry token ids and the output text is empty.
"""

from __future__ import annotations

from pathlib import Path
from typing import Any, Mapping, Sequence


class TokenizerManager:
    def __init__(self, tokenizer: Any) -> None:
        self.tokenizer = tokenizer

    @classmethod
    def from_model_source(cls, source: str | Path) -> "TokenizerManager | None":
        folder = Path(source)
        if not any((folder / name).is_file() for name in ("tokenizer.json", "tokenizer.model",
                                                           "tokenizer_config.json")):
            return None
        from transformers import AutoTokenizer

        return cls(AutoTokenizer.from_pretrained(str(folder), local_files_only=True))

    def encode_messages(self, messages: Sequence[Mapping[str, Any]]) -> list[int]:
        for m in messages:
            if m.get("role") not in ("system", "user", "assistant") or not isinstance(m.get("content"), str):
                raise ValueError("each message needs a role of system/user/assistant and string content")
        ids = self.tokenizer.apply_chat_template(list(messages), add_generation_prompt=True, tokenize=True)
        if isinstance(ids, Mapping):
            ids = ids["input_ids"]
        return [int(t) for t in ids]

    def decode(self, token_ids: Sequence[int]) -> str:
        return self.tokenizer.decode(list(token_ids), skip_special_tokens=True)

    def get_stop_token_ids(self) -> set[int]:
        out: set[int] = set()
        eos = getattr(self.tokenizer, "eos_token_id", None)
        if isinstance(eos, int):
            out.add(eos)
        more = getattr(self.tokenizer, "eos_token_ids", None)
        if isinstance(more, int):
            more = [more]
        for e in more or []:
            out.add(int(e))
        return out
