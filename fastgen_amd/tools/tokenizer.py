"""A model folder's tokenizer, if it has one (``fastgen/utils/tokenizer.py:48-118``):
``tokenizer.json`` through the ``tokenizers`` package, the chat template of
``tokenizer_config.json`` through ``jinja2``."""

from __future__ import annotations

import json
from pathlib import Path
from typing import Dict, List, Optional


class FolderTokenizer:
    def __init__(self, model_dir: str | Path) -> None:
        from tokenizers import Tokenizer

        d = Path(model_dir)
        self.tok = Tokenizer.from_file(str(d / "tokenizer.json"))
        cfg = {}
        if (d / "tokenizer_config.json").is_file():
            with open(d / "tokenizer_config.json") as f:
                cfg = json.load(f)
        self.chat_template: Optional[str] = cfg.get("chat_template")
        self.bos_token = cfg.get("bos_token") if isinstance(cfg.get("bos_token"), str) else None
        eos = cfg.get("eos_token")
        eos = eos.get("content") if isinstance(eos, dict) else eos
        self.eos_token = eos
        eos_id = self.tok.token_to_id(eos) if eos else None
        self.stop_tokens: List[int] = [eos_id] if eos_id is not None else []

    @classmethod
    def maybe(cls, model_dir: str | Path) -> Optional["FolderTokenizer"]:
        return cls(model_dir) if (Path(model_dir) / "tokenizer.json").is_file() else None

    def encode(self, text: str) -> List[int]:
        return self.tok.encode(text, add_special_tokens=False).ids

    def decode(self, ids: List[int]) -> str:
        return self.tok.decode(ids, skip_special_tokens=False)

    def encode_dialog(self, dialog: List[Dict[str, str]]) -> List[int]:
        if self.chat_template:
            import jinja2

            text = jinja2.Environment().from_string(self.chat_template).render(
                messages=dialog, add_generation_prompt=True, bos_token=self.bos_token or "", eos_token=self.eos_token or "")
            return self.encode(text)
        return self.encode("\n".join(m["content"] for m in dialog))
