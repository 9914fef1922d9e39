"""Text in and out of a model folder: tokenizer.json through the `tokenizers` package, the model's own
chat template, the ids that end generation and the folder's sampling defaults.

What the reference's tokenizer does on the request path (src/model/tokenizer/mod.rs):
`encode` runs tokenizer.json's pipeline without adding special tokens and then prepends the
model-declared BOS unless the text already starts with it (:719-737), so a prompt rendered by a chat
template that writes `bos_token` gets exactly one; a one-shot prompt is rendered as a single user
message when the folder declares a template (src/scheduler/mod.rs:1094-1097);
generation ends at the `eos_token_id`(s) of generation_config.json and at special tokens
(tokenizer/mod.rs:710-717); generation_config.json's temperature and top_p stand in for values a
request leaves unset, with `do_sample: false` meaning greedy (:25-27).
"""
from __future__ import annotations

import json
import os
from typing import Dict, List, Optional, Sequence, Tuple


def _read_json(path: str) -> dict:
    try:
        with open(path) as f:
            out = json.load(f)
        return out if isinstance(out, dict) else {}
    except (OSError, ValueError):
        return {}


def _token_text(v) -> Optional[str]:
    """`bos_token` / `eos_token` of tokenizer_config.json: a string or an AddedToken object."""
    if isinstance(v, str):
        return v
    if isinstance(v, dict) and isinstance(v.get("content"), str):
        return v["content"]
    return None


class TextFrontEnd:
    def __init__(self, model_dir: str):
        from tokenizers import Tokenizer
        self.tokenizer = Tokenizer.from_file(os.path.join(model_dir, "tokenizer.json"))
        tc = _read_json(os.path.join(model_dir, "tokenizer_config.json"))
        gc = _read_json(os.path.join(model_dir, "generation_config.json"))
        cfg = _read_json(os.path.join(model_dir, "config.json"))
        self.bos_token = _token_text(tc.get("bos_token"))
        self.eos_token = _token_text(tc.get("eos_token"))
        self.bos_id: Optional[int] = None
        if self.bos_token is not None:
            self.bos_id = self.tokenizer.token_to_id(self.bos_token)
        if self.bos_id is None and isinstance(cfg.get("bos_token_id"), int) and self.bos_token is None:
            self.bos_id = cfg["bos_token_id"]
        template = tc.get("chat_template")
        if isinstance(template, list):                       # several named templates: the default one
            named = {t.get("name"): t.get("template") for t in template if isinstance(t, dict)}
            template = named.get("default")
        self.chat_template: Optional[str] = template if isinstance(template, str) else None
        # ids that end generation: generation_config.json's, config.json's, and the special tokens
        stop = set()
        for src in (gc, cfg):
            ids = src.get("eos_token_id")
            for i in (ids if isinstance(ids, list) else [ids]):
                if isinstance(i, int):
                    stop.add(i)
        vocab = self.tokenizer.get_added_tokens_decoder() if hasattr(self.tokenizer, "get_added_tokens_decoder") else {}
        for i, tok in vocab.items():
            if getattr(tok, "special", False) and i != self.bos_id:
                stop.add(int(i))
        self.stop_ids: Tuple[int, ...] = tuple(sorted(stop))
        # the folder's sampling defaults (None: the engine's)
        self.sampling_defaults: Optional[Tuple[float, float]] = None
        if gc:
            if gc.get("do_sample") is False:
                self.sampling_defaults = (0.0, float(gc.get("top_p", 1.0)))
            elif "temperature" in gc or "top_p" in gc:
                self.sampling_defaults = (float(gc.get("temperature", 1.0)), float(gc.get("top_p", 1.0)))

    def encode(self, text: str) -> List[int]:
        ids = list(self.tokenizer.encode(text, add_special_tokens=False).ids)
        if self.bos_id is not None and (not ids or ids[0] != self.bos_id):
            ids.insert(0, self.bos_id)
        return ids

    def decode(self, ids: Sequence[int]) -> str:
        return self.tokenizer.decode(list(ids))

    def apply_chat_template(self, messages: Sequence[Tuple[str, str]], add_generation_prompt: bool = True,
                            **kwargs) -> str:
        """Renders (role, content) messages with the folder's template, as the usual Python
        implementation does: blocks trimmed, `raise_exception` available, `bos_token` and
        `eos_token` as the folder declares them."""
        if self.chat_template is None:
            raise ValueError("the model folder declares no chat template")
        import jinja2
        from jinja2.sandbox import ImmutableSandboxedEnvironment

        def raise_exception(msg):
            raise jinja2.TemplateError(msg)
        env = ImmutableSandboxedEnvironment(trim_blocks=True, lstrip_blocks=True)
        env.globals["raise_exception"] = raise_exception
        return env.from_string(self.chat_template).render(
            messages=[{"role": r, "content": c} for r, c in messages], add_generation_prompt=add_generation_prompt,
            bos_token=self.bos_token or "", eos_token=self.eos_token or "", **kwargs)

    def prompt_ids(self, prompt: str) -> List[int]:
        """A one-shot prompt: one user message through the template if there is one, else the text."""
        if self.chat_template is not None:
            return self.encode(self.apply_chat_template([("user", prompt)]))
        return self.encode(prompt)


def open_text(model_dir: str) -> Optional[TextFrontEnd]:
    """The folder's text front end, or None when it has no tokenizer.json."""
    if not os.path.isfile(os.path.join(model_dir, "tokenizer.json")):
        return None
    return TextFrontEnd(model_dir)
